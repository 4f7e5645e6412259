"""Tensor.pad / unpad / pad_to_tile / unpad_from_tile (tt_eager/tensor/tensor.cpp:204-260, tensor_impl.cpp:200-283),
tt_lib.tensor.unpad on the device (tt_eager/tt_dnn/op_library/unpad/unpad_op.cpp:95-125) and the BERT-Large matmul
wrappers (tt_eager/tt_dnn/op_library/bmm/bmm_op.cpp:631-742), through the C ABI, bit-exact against the oracle."""
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


def words(t):
    return t._buf.cpu().numpy().view(np.uint32).reshape(-1)


@pytest.mark.parametrize("name", ["BFLOAT8_B", "BFLOAT4_B"])
def test_pad_and_unpad_of_block_float_host_tensors(oracle, name):
    import tt_lib

    dtype = getattr(tt_lib.tensor.DataType, name)
    fmt = int(dtype)
    rng = np.random.default_rng(31)
    shape = (1, 2, 32, 64)
    x = (rng.standard_normal(shape) * np.exp2(rng.integers(-8, 8, size=shape))).astype(np.float32)
    x[0, 1, 5] = 0.0
    x[0, 0, 7, :16] = np.float32(1e-41)                                    # a run of fp32 subnormals: shared exponent 0
    t = tt_lib.tensor.Tensor(torch.from_numpy(x), dtype)                   # declared ROW_MAJOR (pytensor.cpp:145-151)
    assert t.layout == tt_lib.tensor.Layout.ROW_MAJOR
    src = oracle.pack_fp32_vec_as_bfp_tiles(fmt, x.reshape(-1), False)
    assert np.array_equal(words(t), src)
    for out_shape, start, value in (((2, 2, 64, 96), (1, 0, 16, 16), 0.5), ((1, 2, 40, 128), (0, 0, 3, 5), -3.0), ((1, 2, 32, 64), (0, 0, 0, 0), 1.0)):
        p = t.pad(out_shape, start, value)
        assert tuple(p.get_legacy_shape()) == out_shape and p.shape_without_padding() == shape and p.dtype == dtype
        assert np.array_equal(words(p), oracle.pad_bfp(fmt, src, shape, out_shape, start, value)), (out_shape, start)
    for lo, hi in (((0, 0, 0, 0), (0, 1, 15, 63)), ((0, 0, 3, 5), (0, 1, 18, 36)), ((0, 1, 0, 0), (0, 1, 31, 31))):
        u = t.unpad(lo, hi)
        assert tuple(u.get_legacy_shape()) == tuple(h - l + 1 for l, h in zip(lo, hi))
        assert np.array_equal(words(u), oracle.unpad_bfp(fmt, src, shape, lo, hi)), (lo, hi)
    with pytest.raises(RuntimeError, match="whole tiles"):
        t.unpad((0, 0, 0, 0), (0, 0, 15, 30))
    with pytest.raises(RuntimeError, match="input_tensor_start"):
        t.pad((1, 2, 32, 64), (0, 0, 1, 0), 0.0)
    # pad_to_tile / unpad_from_tile on a ragged tensor (volume must still be whole chunks: 2 x 16 x 32)
    small = tt_lib.tensor.Tensor(torch.from_numpy(x[:, :, :16, :32].copy()), dtype)
    tiled = small.pad_to_tile(0.0)
    assert tuple(tiled.get_legacy_shape()) == (1, 2, 32, 32)
    ssrc = oracle.pack_fp32_vec_as_bfp_tiles(fmt, x[:, :, :16, :32].reshape(-1), False)
    assert np.array_equal(words(tiled), oracle.pad_bfp(fmt, ssrc, (1, 2, 16, 32), (1, 2, 32, 32), (0, 0, 0, 0), 0.0))
    back = tiled.unpad_from_tile((1, 2, 16, 32))
    assert np.array_equal(words(back), oracle.unpad_bfp(fmt, words(tiled), (1, 2, 32, 32), (0, 0, 0, 0), (0, 1, 15, 31)))


@pytest.mark.parametrize("torch_dtype", [torch.bfloat16, torch.float32, torch.int32])
def test_pad_and_unpad_of_dense_host_tensors(oracle, torch_dtype):
    import tt_lib

    torch.manual_seed(32)
    x = (torch.randn(2, 3, 5, 7) * 50).to(torch_dtype)
    t = tt_lib.tensor.Tensor(x)
    view = {torch.bfloat16: np.uint16, torch.float32: np.float32, torch.int32: np.uint32}[torch_dtype]
    raw = x.view(torch.int16).numpy().view(np.uint16) if torch_dtype == torch.bfloat16 else x.numpy().view(view)
    pad_value = 2.7182817     # a bfloat16 keeps its upper 16 bits (tt_metal/common/bfloat16.hpp:28-38), an integer its integral part
    fill = {torch.bfloat16: np.uint16(np.float32(pad_value).view(np.uint32) >> 16), torch.float32: np.float32(pad_value), torch.int32: np.uint32(2)}[torch_dtype]
    p = t.pad((3, 4, 8, 10), (1, 0, 2, 3), pad_value)
    got = p._buf.view(torch.int16).numpy().view(np.uint16) if torch_dtype == torch.bfloat16 else p._buf.numpy().view(view)
    want = oracle.pad_rowmajor(raw, (3, 4, 8, 10), (1, 0, 2, 3), fill)
    assert got.shape == (3, 4, 8, 10) and np.array_equal(got.view(np.uint8), want.view(np.uint8))
    u = p.unpad((1, 0, 2, 3), (2, 2, 6, 9))
    assert torch.equal(u.to_torch(), x)
    assert tuple(t.pad_to_tile(0.0).get_legacy_shape()) == (2, 3, 32, 32)
    assert torch.equal(t.pad_to_tile(0.0).unpad_from_tile((2, 3, 5, 7)).to_torch(), x)
    with pytest.raises(RuntimeError, match="Device storage"):
        t.to(tt_lib.device.CreateDevice(0)).pad((3, 4, 8, 10), (0, 0, 0, 0), 0.0)


@pytest.mark.parametrize("name", ["bfloat16", "bfloat8_b", "bfloat4_b"])
def test_unpad_on_device_moves_whole_tiles(oracle, device, name):
    import tt_lib
    import ttnn

    dtype = getattr(ttnn, name)
    torch.manual_seed(33)
    x = torch.randn(2, 3, 96, 160).to(torch.bfloat16)
    t = ttnn.from_torch(x, dtype=dtype, layout=ttnn.TILE_LAYOUT, device=device)
    full = ttnn.to_torch(t)
    part = tt_lib.tensor.unpad(t, (1, 0, 32, 64), (1, 1, 95, 127))
    assert tuple(part.get_legacy_shape()) == (1, 2, 64, 64) and part.dtype == dtype and part.layout == ttnn.TILE_LAYOUT
    assert torch.equal(ttnn.to_torch(part), full[1:2, 0:2, 32:96, 64:128])
    per_tile = {"bfloat16": 1024, "bfloat8_b": 272, "bfloat4_b": 144}[name]
    assert torch.equal(part._buf.view(1, 2, 2, 2, per_tile), t._buf.view(2, 3, 3, 5, per_tile)[1:2, 0:2, 1:3, 2:4])
    with pytest.raises(RuntimeError, match="full tiles"):
        tt_lib.tensor.unpad(t, (0, 0, 16, 0), (0, 0, 47, 31))
    rm = ttnn.from_torch(x, layout=ttnn.ROW_MAJOR_LAYOUT, device=device)
    cut = tt_lib.tensor.unpad(rm, (0, 1, 5, 8), (1, 2, 50, 17))
    assert torch.equal(ttnn.to_torch(cut), x[0:2, 1:3, 5:51, 8:18])
    with pytest.raises(RuntimeError, match="packable"):
        tt_lib.tensor.unpad(rm, (0, 0, 0, 1), (0, 0, 0, 4))


def test_bert_large_matmuls(oracle, device):
    import tt_lib
    import ttnn

    torch.manual_seed(34)
    ttl = tt_lib.tensor

    def packed(w, dtype=ttnn.bfloat8_b):
        return ttnn.from_torch(w, dtype=dtype, layout=ttnn.TILE_LAYOUT, device=device)

    def quantised(w):
        x = w.float().numpy().reshape((-1,) + tuple(w.shape[-2:]))
        return torch.from_numpy(oracle.to_torch_bfp_tiles(3, oracle.from_torch_bfp_tiles(3, x), x.shape)).reshape(w.shape).double()

    def close(got, want, k):
        got, want = ttnn.to_torch(got).double(), want
        assert got.shape == want.shape
        assert float(torch.corrcoef(torch.stack([got.reshape(-1), want.reshape(-1)]))[0, 1]) >= 0.9999
        assert torch.all((got - want).abs() <= 2.0 ** -8 * want.abs() + 1e-2 * k ** 0.5 * 2.0 ** -8)

    a = torch.randn(2, 1, 384, 1024).to(torch.bfloat16)
    ta = ttnn.from_torch(a, layout=ttnn.TILE_LAYOUT, device=device)
    for fn, n, kwargs in ((ttl.bert_large_fused_qkv_matmul, 3072, {}), (ttl.bert_large_selfout_matmul, 1024, {}),
                          (ttl.bert_large_ff1_matmul, 4096, {"fused_activation": [ttl.FusibleActivation.GELU, True]})):
        w = torch.randn(1, 1, 1024, n) * 0.02
        bias = (torch.randn(1, 1, 1, n) * 0.1).to(torch.bfloat16)
        tb = ttnn.from_torch(bias.expand(1, 1, 32, n).contiguous(), layout=ttnn.TILE_LAYOUT, device=device)
        out = fn(ta, packed(w), tb, **kwargs)
        want = a.double() @ quantised(w) + bias.double()
        close(out, torch.nn.functional.gelu(want) if kwargs else want, 1024)
        with pytest.raises(RuntimeError, match="Unsupported input shape"):
            fn(ta, packed(torch.randn(1, 1, 1024, n + 32)))
    a2 = torch.randn(1, 1, 384, 4096).to(torch.bfloat16)
    w2 = torch.randn(1, 1, 4096, 1024) * 0.02
    close(ttl.bert_large_ff2_matmul(ttnn.from_torch(a2, layout=ttnn.TILE_LAYOUT, device=device), packed(w2)), a2.double() @ quantised(w2), 4096)
    q = torch.randn(1, 16, 384, 64).to(torch.bfloat16)
    kt = torch.randn(1, 16, 64, 384)
    close(ttl.bert_large_pre_softmax_bmm(ttnn.from_torch(q, layout=ttnn.TILE_LAYOUT, device=device), packed(kt)), q.double() @ quantised(kt), 64)
    p = torch.rand(1, 16, 384, 384).to(torch.bfloat16)
    v = torch.randn(1, 16, 384, 64)
    close(ttl.bert_large_post_softmax_bmm(ttnn.from_torch(p, layout=ttnn.TILE_LAYOUT, device=device), packed(v)), p.double() @ quantised(v), 384)
    with pytest.raises(RuntimeError, match="Unsupported input shape"):
        ttl.bert_large_pre_softmax_bmm(ttnn.from_torch(p, layout=ttnn.TILE_LAYOUT, device=device), packed(v))
