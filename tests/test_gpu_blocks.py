"""Callers either side of the block-float GEMMs, on the GPU: elementwise ops (ttnn.mul and friends), weight caches as tensor
files, and the Falcon-7B / Mistral-7B MLP blocks, in the shape of the reference's own tests
(tests/ttnn/integration_tests/falcon7b/test_falcon_mlp.py:17-95, tests/ttnn/unit_tests/test_as_tensor.py,
tests/ttnn/unit_tests/test_dump_and_load.py, tests/ttnn/unit_tests/operations/test_mul.py).

Block parity (stated here, the reference's own bar is PCC >= 0.985 against the torch model with unquantised weights):
PCC >= 0.9999 against an fp64 evaluation that uses the weights as the oracle unpacks them and rounds the activations
between the GEMMs to bf16 as the device does; PCC >= 0.99 against the plain torch functional model.
"""
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


def pcc(a, b):
    a, b = a.double().reshape(-1), b.double().reshape(-1)
    return float(torch.corrcoef(torch.stack([a, b]))[0, 1])


def quantised(oracle, ttnn_dtype, w):
    """[K, N] fp32 -> the values a block-float tensor of it holds (oracle pack + unpack), fp64."""
    x = w.float().numpy()[None]
    words = oracle.from_torch_bfp_tiles(int(ttnn_dtype), x)
    return torch.from_numpy(oracle.to_torch_bfp_tiles(int(ttnn_dtype), words, x.shape)[0]).double()


def bf16_round(x):
    return x.float().to(torch.bfloat16).double()


# ---- elementwise ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(32, 64), (1, 1, 32, 18176), (2, 3, 64, 96), (7, 3)])
@pytest.mark.parametrize("layout_name", ["TILE_LAYOUT", "ROW_MAJOR_LAYOUT"])
def test_binary_ops_match_torch_bf16(device, shape, layout_name):
    import ttnn

    layout = getattr(ttnn, layout_name)
    torch.manual_seed(11)
    a = torch.randn(shape).to(torch.bfloat16)
    b = torch.randn(shape).to(torch.bfloat16)
    ta = ttnn.from_torch(a, layout=layout, device=device)
    tb = ttnn.from_torch(b, layout=layout, device=device)
    for fn, ref in ((ttnn.mul, torch.mul), (ttnn.add, torch.add), (ttnn.sub, torch.sub)):
        out = fn(ta, tb)
        assert out.shape == shape and out.dtype == ttnn.bfloat16 and out.layout == layout
        want = ref(a.float(), b.float()).to(torch.bfloat16)         # fp32 arithmetic, one rounding: what torch does for bf16 too
        assert torch.equal(ttnn.to_torch(out), want)
    assert torch.equal(ttnn.to_torch(ttnn.mul(ta, 0.5)), (a.float() * 0.5).to(torch.bfloat16))
    assert torch.equal(ttnn.to_torch(ttnn.multiply(ta, tb)), torch.mul(a.float(), b.float()).to(torch.bfloat16))


def test_unary_ops(device):
    import ttnn

    torch.manual_seed(12)
    a = (torch.randn(1, 1, 64, 160) * 3).to(torch.bfloat16)
    ta = ttnn.from_torch(a, layout=ttnn.TILE_LAYOUT, device=device)
    for fn, ref in ((ttnn.gelu, torch.nn.functional.gelu), (ttnn.relu, torch.relu), (ttnn.silu, torch.nn.functional.silu)):
        got = ttnn.to_torch(fn(ta)).float()
        want = ref(a.double())
        assert torch.allclose(got.double(), want, rtol=2 ** -8, atol=1e-6)


def test_block_float_operand_and_errors(oracle, device):
    import ttnn

    torch.manual_seed(13)
    a = torch.randn(64, 64)
    b = torch.randn(64, 64).to(torch.bfloat16)
    ta = ttnn.from_torch(a, dtype=ttnn.bfloat8_b, layout=ttnn.TILE_LAYOUT, device=device)
    tb = ttnn.from_torch(b, layout=ttnn.TILE_LAYOUT, device=device)
    out = ttnn.mul(ta, tb)
    assert out.dtype == ttnn.bfloat8_b                              # the output takes input a's dtype
    aq = quantised(oracle, ttnn.bfloat8_b, a)
    product = (aq.float() * b.float()).to(torch.bfloat16).float()
    want = oracle.to_torch_bfp_tiles(3, oracle.from_torch_bfp_tiles(3, product.numpy()[None]), (1, 64, 64))[0]
    assert np.array_equal(ttnn.to_torch(out).numpy(), want)
    with pytest.raises(RuntimeError, match="on device"):
        ttnn.mul(ttnn.from_torch(b, layout=ttnn.TILE_LAYOUT), tb)
    with pytest.raises(RuntimeError, match="broadcast"):
        ttnn.mul(tb, ttnn.from_torch(b[:1], layout=ttnn.ROW_MAJOR_LAYOUT, device=device))
    with pytest.raises(TypeError):
        ttnn.mul(tb, "x")


# ---- tensor files and weight caches -----------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["bfloat8_b", "bfloat4_b", "bfloat16"])
def test_dump_and_load_tilized(tmp_path, device, name):
    import ttnn

    dtype = getattr(ttnn, name)
    torch.manual_seed(14)
    x = torch.rand((96, 160), dtype=torch.float32).to(torch.bfloat16)
    t = ttnn.from_torch(x, dtype=dtype, layout=ttnn.TILE_LAYOUT)
    ttnn.dump_tensor(tmp_path / "tensor.bin", t)
    assert (tmp_path / "tensor.bin").stat().st_size == 200 + 15 * {"bfloat8_b": 1088, "bfloat4_b": 576, "bfloat16": 2048}[name]
    loaded = ttnn.load_tensor(tmp_path / "tensor.bin")
    assert loaded.dtype == dtype and loaded.layout == ttnn.TILE_LAYOUT and loaded.shape == t.shape
    assert torch.equal(loaded._buf, t._buf)
    assert torch.equal(ttnn.to_torch(loaded), ttnn.to_torch(t))
    with pytest.raises(RuntimeError, match="Device storage"):
        ttnn.dump_tensor(tmp_path / "d.bin", ttnn.to_device(t, device))


def test_as_tensor_with_cache(tmp_path, device):
    """tests/ttnn/unit_tests/test_as_tensor.py:25-58, with a block-float weight."""
    import ttnn

    torch.manual_seed(15)
    w = torch.rand((7, 3), dtype=torch.float32)
    plain = ttnn.as_tensor(w.to(torch.bfloat16), layout=ttnn.TILE_LAYOUT, device=device, memory_config=ttnn.L1_MEMORY_CONFIG)
    assert torch.allclose(ttnn.to_torch(plain), w.to(torch.bfloat16))
    big = torch.randn(160, 96)
    first = ttnn.as_tensor(big, dtype=ttnn.bfloat8_b, layout=ttnn.TILE_LAYOUT, device=device, cache_file_name=tmp_path / "sub" / "w")
    file = tmp_path / "sub" / "w_dtype_BFLOAT8_B_layout_TILE.bin"
    assert file.exists() and first.dtype == ttnn.bfloat8_b and first.layout == ttnn.TILE_LAYOUT and first.device() == device
    second = ttnn.as_tensor(torch.zeros_like(big), dtype=ttnn.bfloat8_b, layout=ttnn.TILE_LAYOUT, device=device, cache_file_name=tmp_path / "sub" / "w")
    assert torch.equal(second._buf, first._buf)                    # taken from the file, not from the (different) torch tensor
    assert ttnn.is_tensor_storage_on_device(second)


# ---- MLP blocks -------------------------------------------------------------------------------------------------------
# The decode MLPs of the two models, issued op by op on the mirrored API; what is checked against is the torch functional
# model of tests/ttnn/integration_tests/falcon7b/test_falcon_mlp.py:17-44 (and its Mistral counterpart), evaluated in fp64.
def weight_on_device(ttnn, device, linear_weight, dtype, cache_file_name=None):
    """torch.nn.Linear weight [out, in] -> [1, 1, in, out] block-float tiles on the device (through a weight cache file when named)."""
    return ttnn.as_tensor(linear_weight.t().contiguous()[None, None], dtype=dtype, layout=ttnn.TILE_LAYOUT, device=device,
                          cache_file_name=cache_file_name)


def falcon_mlp_on_device(tt_lib, x, w_up, w_down):
    gelu = [tt_lib.tensor.FusibleActivation.GELU, True]
    return tt_lib.tensor.falcon_dense_4h_to_h_matmul(tt_lib.tensor.falcon_dense_h_to_4h_matmul(x, w_up, fused_activation=gelu), w_down)


def mistral_mlp_on_device(ttnn, x, w_gate, w_up, w_down):
    return ttnn.linear(ttnn.mul(ttnn.linear(x, w_gate, activation="silu"), ttnn.linear(x, w_up)), w_down)


@pytest.mark.parametrize("seq,hidden", [(32, 128), (128, 256), (32, 4544)])
def test_falcon_mlp_block(oracle, device, tmp_path, seq, hidden):
    import tt_lib
    import ttnn

    torch.manual_seed(0)
    up, down = torch.randn(4 * hidden, hidden) * 0.02, torch.randn(hidden, 4 * hidden) * 0.02
    x = ((torch.rand(1, 1, seq, hidden) * 2) - 1).to(torch.bfloat16)
    cache = tmp_path if hidden <= 256 else None
    w_up = weight_on_device(ttnn, device, up, ttnn.bfloat8_b, cache and cache / "up")
    w_down = weight_on_device(ttnn, device, down, ttnn.bfloat8_b, cache and cache / "down")
    assert w_up.dtype == tt_lib.tensor.DataType.BFLOAT8_B
    out = falcon_mlp_on_device(tt_lib, ttnn.from_torch(x, dtype=ttnn.bfloat16, layout=ttnn.TILE_LAYOUT, device=device), w_up, w_down)
    assert tuple(out.shape) == (1, 1, seq, hidden) and out.dtype == ttnn.bfloat16
    got = ttnn.to_torch(out)[0, 0]
    hidden_act = bf16_round(torch.nn.functional.gelu(x[0, 0].double() @ quantised(oracle, ttnn.bfloat8_b, up.t())))
    assert pcc(got, hidden_act @ quantised(oracle, ttnn.bfloat8_b, down.t())) >= 0.9999
    assert pcc(got, torch.nn.functional.gelu(x[0, 0].float() @ up.t()) @ down.t()) >= 0.99      # unquantised weights
    if cache is not None:                                              # a second conversion reads the cached tensor file
        again = weight_on_device(ttnn, device, torch.zeros_like(down), ttnn.bfloat8_b, cache / "down")
        assert torch.equal(again._buf, w_down._buf)


@pytest.mark.parametrize("seq,dim,hidden_dim,name", [(32, 128, 352, "bfloat8_b"), (64, 256, 704, "bfloat4_b"), (32, 4096, 14336, "bfloat4_b")])
def test_mistral_mlp_block(oracle, device, seq, dim, hidden_dim, name):
    import ttnn

    dtype = getattr(ttnn, name)
    torch.manual_seed(1)
    gate, up, down = torch.randn(hidden_dim, dim) * 0.02, torch.randn(hidden_dim, dim) * 0.02, torch.randn(dim, hidden_dim) * 0.02
    x = torch.randn(1, 1, seq, dim).to(torch.bfloat16)
    out = mistral_mlp_on_device(ttnn, ttnn.from_torch(x, dtype=ttnn.bfloat16, layout=ttnn.TILE_LAYOUT, device=device),
                                *(weight_on_device(ttnn, device, w, dtype) for w in (gate, up, down)))
    assert tuple(out.shape) == (1, 1, seq, dim)
    got = ttnn.to_torch(out)[0, 0]
    xd = x[0, 0].double()
    gated = bf16_round(torch.nn.functional.silu(xd @ quantised(oracle, dtype, gate.t())))
    want_q = bf16_round(gated * bf16_round(xd @ quantised(oracle, dtype, up.t()))) @ quantised(oracle, dtype, down.t())
    assert pcc(got, want_q) >= 0.9999
    want = (torch.nn.functional.silu(x[0, 0].float() @ gate.t()) * (x[0, 0].float() @ up.t())) @ down.t()
    assert pcc(got, want) >= (0.99 if name == "bfloat8_b" else 0.95)   # 3-bit mantissas: the quantisation itself costs that much


@pytest.mark.parametrize("seq,dim,hidden_dim,name", [(32, 128, 352, "bfloat8_b"), (32, 4096, 14336, "bfloat4_b")])
def test_gated_linear_is_linear_linear_mul_in_one_launch(oracle, device, seq, dim, hidden_dim, name):
    """ttnn.experimental.gated_linear(x, w1, w3) against what a gated MLP issues on the reference's surface: ttnn.linear(x, w1,
    activation="silu"), ttnn.linear(x, w3), ttnn.mul.  The fused launch multiplies the two fp32 sums and rounds once, the three
    ops round each factor to bf16 first: equal within two bf16 roundings, and both within the quantised model's PCC."""
    import ttnn

    dtype = getattr(ttnn, name)
    torch.manual_seed(2)
    gate, up = torch.randn(hidden_dim, dim) * 0.02, torch.randn(hidden_dim, dim) * 0.02
    x = torch.randn(1, 1, seq, dim).to(torch.bfloat16)
    tx = ttnn.from_torch(x, dtype=ttnn.bfloat16, layout=ttnn.TILE_LAYOUT, device=device)
    w1, w3 = (weight_on_device(ttnn, device, w, dtype) for w in (gate, up))
    fused = ttnn.experimental.gated_linear(tx, w1, w3, activation="silu")
    assert tuple(fused.shape) == (1, 1, seq, hidden_dim) and fused.dtype == ttnn.bfloat16 and fused.layout == ttnn.TILE_LAYOUT
    three = ttnn.mul(ttnn.linear(tx, w1, activation="silu"), ttnn.linear(tx, w3))
    got, ops = ttnn.to_torch(fused)[0, 0].double(), ttnn.to_torch(three)[0, 0].double()
    xd = x[0, 0].double()
    want = torch.nn.functional.silu(xd @ quantised(oracle, dtype, gate.t())) * (xd @ quantised(oracle, dtype, up.t()))
    assert pcc(got, want) >= 0.9999 and pcc(ops, want) >= 0.9999
    assert torch.all((got - ops).abs() <= 2.0 ** -6 * want.abs() + 1e-6)
    with pytest.raises(RuntimeError, match="same dtype and shape"):
        ttnn.experimental.gated_linear(tx, w1, weight_on_device(ttnn, device, up[:32], dtype))
    with pytest.raises(RuntimeError, match="is not supported as activation"):
        ttnn.experimental.gated_linear(tx, w1, w3, activation="tanh")


# ---- device-resident dtype changes ------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["bfloat8_b", "bfloat4_b"])
def test_to_layout_with_dtype_and_clone(oracle, device, name):
    """ttnn.to_layout(.., TILE_LAYOUT, dtype=) on a bf16 device tensor (ttnn/ttnn/operations/core.py:684-711) and ttnn.clone
    (core.py:819-839).  The Tensix packer's rounding is not pinned by the sources at hand; checked here: the result is the
    reference's HOST packer applied once to the tile-ordered values (parity with the device op itself: unpinned)."""
    import ttnn

    dtype = getattr(ttnn, name)
    fmt = int(dtype)
    torch.manual_seed(21)
    x = torch.randn(2, 64, 96).to(torch.bfloat16)
    t = ttnn.from_torch(x, layout=ttnn.ROW_MAJOR_LAYOUT, device=device)
    packed = ttnn.to_layout(t, ttnn.TILE_LAYOUT, dtype=dtype)
    assert packed.dtype == dtype and packed.layout == ttnn.TILE_LAYOUT and ttnn.is_tensor_storage_on_device(packed)
    tiles = oracle.tilize_nchw_4faces(x.float().numpy()[None])
    want = oracle.pack_fp32_vec_as_bfp_tiles(fmt, tiles, False)
    assert np.array_equal(packed._buf.cpu().numpy().view(np.uint32), want)
    # clone: bf16 tiles -> block-float gives the same words; block-float -> bf16 gives the unpacked values exactly
    tiled = ttnn.to_layout(t, ttnn.TILE_LAYOUT)
    cloned = ttnn.clone(tiled, ttnn.DRAM_MEMORY_CONFIG, dtype)
    assert cloned.layout == ttnn.TILE_LAYOUT and torch.equal(cloned._buf, packed._buf)
    back = ttnn.clone(cloned, ttnn.DRAM_MEMORY_CONFIG, ttnn.bfloat16)
    assert back.dtype == ttnn.bfloat16 and torch.equal(ttnn.to_torch(back).float(), ttnn.to_torch(cloned))
    same = ttnn.clone(tiled, ttnn.DRAM_MEMORY_CONFIG, None)
    assert same.dtype == ttnn.bfloat16 and torch.equal(same._buf, tiled._buf) and same._buf.data_ptr() != tiled._buf.data_ptr()
    with pytest.raises(RuntimeError, match="Unsupported datatype conversion"):
        ttnn.to_layout(ttnn.from_torch(x, layout=ttnn.ROW_MAJOR_LAYOUT), ttnn.TILE_LAYOUT, dtype=dtype)       # not on the device
    with pytest.raises(RuntimeError, match="Unsupported datatype conversion"):
        ttnn.to_layout(tiled, ttnn.ROW_MAJOR_LAYOUT, dtype=dtype)
    with pytest.raises(RuntimeError, match="on device"):
        ttnn.clone(ttnn.from_torch(x), ttnn.DRAM_MEMORY_CONFIG, dtype)


@pytest.mark.parametrize("name", ["bfloat16", "bfloat8_b", "bfloat4_b"])
def test_getitem_prefix_on_device(oracle, device, name):
    """ttnn.Tensor.__getitem__ (ttnn/ttnn/operations/core.py:56-114): a prefix of a device tensor keeps whole tiles, so a
    block-float result equals the corresponding tiles of the source, and its values equal the torch slice of the source's."""
    import ttnn

    dtype = getattr(ttnn, name)
    torch.manual_seed(22)
    x = torch.randn(2, 3, 96, 160).to(torch.bfloat16)
    t = ttnn.from_torch(x, dtype=dtype, layout=ttnn.TILE_LAYOUT, device=device)
    full = ttnn.to_torch(t)
    part = t[:1, :2, :40, :70]
    assert tuple(part.shape) == (1, 2, 40, 70) and tuple(part.shape.with_tile_padding()) == (1, 2, 64, 96)
    assert part.dtype == dtype and part.layout == ttnn.TILE_LAYOUT and ttnn.is_tensor_storage_on_device(part)
    assert torch.equal(ttnn.to_torch(part), full[:1, :2, :40, :70])
    if name != "bfloat16":      # the tiles themselves: tile (r, c) of slice (0, ch) of the source
        per_tile = {"bfloat8_b": 272, "bfloat4_b": 144}[name]
        src = t._buf.view(2, 3, 3, 5, per_tile)
        assert torch.equal(part._buf.view(1, 2, 2, 3, per_tile), src[:1, :2, :2, :3])
    assert t[:2] is not None and tuple(t[:2].shape) == (2, 3, 96, 160)
    row_major = ttnn.from_torch(x, layout=ttnn.ROW_MAJOR_LAYOUT, device=device)
    assert torch.equal(ttnn.to_torch(row_major[:2, :1, :5, :9]), x[:2, :1, :5, :9])
    with pytest.raises(RuntimeError, match="cannot slice"):
        t[:, :, 32:64, :]
    with pytest.raises(RuntimeError, match="cannot slice"):
        ttnn.from_torch(x, layout=ttnn.ROW_MAJOR_LAYOUT)[:1]
    with pytest.raises(RuntimeError, match="Too many slices"):
        t[:1, :1, :1, :1, :1]
