"""Pins the oracle's tilize/untilize and gold matmul (no GPU)."""
import numpy as np
import pytest

from ttmi import workloads


def closed_form_tilize_index(n, c, h, w):
    """dst index of every element of a [n,c,h,w] tensor (h, w multiples of 32) in 4-face tile order.

    tile = ((b*(h/32) + r/32)*(w/32) + col/32, face = 2*((r%32)/16) + (col%32)/16,
    dst = tile*1024 + face*256 + (r%16)*16 + col%16  — the layout drawn in
    tt_metal/common/test_tiles.hpp:18-22 and walked by tilize_untilize.hpp:44-53.
    """
    b, r, col = np.meshgrid(np.arange(n * c), np.arange(h), np.arange(w), indexing="ij")
    tile = (b * (h // 32) + r // 32) * (w // 32) + col // 32
    face = 2 * ((r % 32) // 16) + (col % 32) // 16
    return tile * 1024 + face * 256 + (r % 16) * 16 + col % 16


@pytest.mark.parametrize("shape", [(2, 3, 64, 96), (1, 1, 32, 32), (1, 4, 96, 32)])
def test_tilize_is_the_closed_form_permutation(oracle, shape):
    n, c, h, w = shape
    x = np.arange(n * c * h * w, dtype=np.float32).reshape(shape)
    want = np.empty(x.size, dtype=np.float32)
    want[closed_form_tilize_index(n, c, h, w).reshape(-1)] = x.reshape(-1)
    got = oracle.tilize_nchw_4faces(x)
    assert np.array_equal(got, want)
    assert np.array_equal(oracle.untilize_nchw_4faces(got, shape), x)
    # the bf16 tilizer of tilize_untilize.hpp gives the same order (blocks of h x w)
    u16 = (np.arange(x.size) % 65521).astype(np.uint16)
    want16 = np.empty_like(u16)
    want16[closed_form_tilize_index(n, c, h, w).reshape(-1)] = u16
    assert np.array_equal(oracle.tilize_bf16_blocks(u16, h, w), want16)
    assert np.array_equal(oracle.untilize_bf16_blocks(want16, h, w), u16)


def test_tilize_zero_pads_ragged_shapes(oracle):
    x = np.arange(1, 2 * 5 * 40 + 1, dtype=np.float32).reshape(1, 2, 5, 40)
    got = oracle.tilize_nchw_4faces(x)
    padded = np.zeros((1, 2, 32, 64), dtype=np.float32)
    padded[:, :, :5, :40] = x
    assert np.array_equal(got, oracle.tilize_nchw_4faces(padded))
    assert np.count_nonzero(got) == x.size


def test_tilize_untilize_identity_sweep(oracle):
    """tests/tt_metal/tt_metal/unit_tests/host_apis/test_tilize_untilize.cpp:9-47: batches x tiles sweep."""
    rng = np.random.default_rng(2)
    for nb in (1, 2, 8):
        for rt in (1, 3, 8):
            for ct in (1, 2, 8):
                m, n = rt * 32, ct * 32
                v = rng.integers(0, 65536, size=nb * m * n).astype(np.uint16)
                t = oracle.tilize_bf16_blocks(v, m, n)
                assert np.array_equal(oracle.untilize_bf16_blocks(t, m, n), v)
                assert np.array_equal(t, oracle.tilize_nchw_4faces(v.reshape(1, nb, m, n)))


def test_tilize_rejects_bad_shapes(oracle):
    """test_tilize_untilize.cpp:49-97: zero sizes, non-divisible sizes and non-multiples of 32 fail."""
    v = np.zeros(1024, dtype=np.uint16)
    for m, n in [(0, 32), (32, 0), (32, 33), (16, 64), (64, 32)]:
        if m * n == 2048:
            with pytest.raises(RuntimeError):
                oracle.tilize_bf16_blocks(v[:1000], m, n)
            continue
        with pytest.raises(RuntimeError):
            oracle.tilize_bf16_blocks(v, m, n)
        with pytest.raises(RuntimeError):
            oracle.untilize_bf16_blocks(v, m, n)


def test_bf16_truncation(oracle):
    # bfloat16.hpp:28-38 keeps the upper half of the word
    for val, want in [(1.0, 0x3F80), (1.00390625, 0x3F80), (-2.5, 0xC020), (3.14159274, 0x4049)]:
        assert oracle.lib().oracle_bf16_truncate(val) == want


def test_gold_bmm_exact_on_small_integers_and_close_to_float64(oracle):
    rng = np.random.default_rng(4)
    nb, m, k, n = 2, 5, 48, 7
    a = rng.integers(-8, 9, size=(nb, m, k)).astype(np.float32)
    b = rng.integers(-8, 9, size=(nb, k, n)).astype(np.float32)
    f, h = oracle.gold_bmm(oracle.bf16_truncate(a), oracle.bf16_truncate(b), nb, m, k, n)
    assert np.array_equal(f, np.matmul(a.astype(np.int64), b.astype(np.int64)).astype(np.float32))
    assert np.array_equal(h, oracle.bf16_truncate(f))
    a = workloads.bf16_bits_to_f32(workloads.activations_bf16(m, k, 1, batch=nb))
    b = workloads.bf16_bits_to_f32(workloads.f32_to_bf16_bits_rne(workloads.weights_f32(k, n, 2, batch=nb)))
    f, _ = oracle.gold_bmm(oracle.bf16_truncate(a), oracle.bf16_truncate(b), nb, m, k, n)
    exact = np.matmul(a.astype(np.float64), b.astype(np.float64))
    bound = k * 2.0 ** -24 * np.matmul(np.abs(a).astype(np.float64), np.abs(b).astype(np.float64))
    assert np.all(np.abs(f - exact) <= bound + 1e-30)
    assert np.array_equal(oracle.matmul_reference(a[0], b[0]), exact[0].astype(np.float32))


# ---- pad / unpad (tt_eager/tensor/tensor_impl.hpp:508-660, tensor_impl.cpp:200-283) -------------------------------------
@pytest.mark.parametrize("dtype", [np.float32, np.uint16, np.uint32])
def test_pad_and_unpad_rowmajor_are_numpy_pad_and_slicing(oracle, dtype):
    """The reference writes the output front to back with runs of the pad value; numpy.pad and basic slicing state the same
    result without any of its index arithmetic (a wrong stride, a swapped front / back pad or an off-by-one end fails here)."""
    rng = np.random.default_rng(5)
    x = rng.integers(1, 60000, size=(2, 3, 5, 7)).astype(dtype)
    out_shape, start = (4, 5, 9, 16), (1, 2, 3, 4)
    want = np.pad(x, [(s, o - s - i) for s, o, i in zip(start, out_shape, x.shape)], constant_values=dtype(9))
    assert np.array_equal(oracle.pad_rowmajor(x, out_shape, start, 9), want)
    assert np.array_equal(oracle.pad_rowmajor(x, x.shape, (0, 0, 0, 0), 9), x)
    lo, hi = (1, 0, 2, 3), (1, 2, 4, 6)
    assert np.array_equal(oracle.unpad_rowmajor(x, lo, hi), x[1:2, 0:3, 2:5, 3:7])
    assert np.array_equal(oracle.unpad_rowmajor(want, start, tuple(s + i - 1 for s, i in zip(start, x.shape))), x)   # unpad inverts pad
    with pytest.raises(RuntimeError):
        oracle.pad_rowmajor(x, (2, 3, 5, 7), (0, 0, 0, 1), 0)
    with pytest.raises(RuntimeError):
        oracle.unpad_rowmajor(x, (0, 0, 0, 0), (1, 2, 4, 7))


@pytest.mark.parametrize("fmt", [3, 4])
def test_pad_and_unpad_block_float_requantise_the_moved_values(oracle, fmt):
    """pad_bfloat8_b / unpad_bfloat8_b: unpack -> fp32 pad / unpad -> pack.  Checked against numpy.pad / slicing of the
    unpacked values followed by one sequential pack; and, where the window keeps every 16-element run intact, against the
    source's own codes (nothing is re-quantised when a run moves as a whole)."""
    rng = np.random.default_rng(6)
    shape = (1, 2, 32, 64)
    x = (rng.standard_normal(shape) * np.exp2(rng.integers(-6, 6, size=shape))).astype(np.float32)
    words = oracle.pack_fp32_vec_as_bfp_tiles(fmt, x.reshape(-1), False)
    values = oracle.unpack_bfp_tiles_into_float_vec(fmt, words, False).reshape(shape)
    out_shape, start = (2, 2, 64, 96), (1, 0, 16, 16)
    padded = np.pad(values, [(s, o - s - i) for s, o, i in zip(start, out_shape, shape)], constant_values=np.float32(0.5))
    got = oracle.pad_bfp(fmt, words, shape, out_shape, start, 0.5)
    assert np.array_equal(got, oracle.pack_fp32_vec_as_bfp_tiles(fmt, padded.reshape(-1), False))
    # every run of 16 stays whole here (offsets are multiples of 16), so unpacking gives back exactly the padded values
    assert np.array_equal(oracle.unpack_bfp_tiles_into_float_vec(fmt, got, False).reshape(out_shape), padded)
    lo, hi = (0, 1, 3, 5), (0, 1, 18, 36)                                   # 16 x 32 values = half a chunk: rejected
    with pytest.raises(RuntimeError):
        oracle.unpad_bfp(fmt, words, shape, lo, hi)
    lo, hi = (0, 0, 3, 5), (0, 1, 18, 36)                                   # 2 x 16 x 32 = one chunk, runs cut at column 5
    cut = oracle.unpad_bfp(fmt, words, shape, lo, hi)
    assert np.array_equal(cut, oracle.pack_fp32_vec_as_bfp_tiles(fmt, values[0:1, 0:2, 3:19, 5:37].reshape(-1), False))
    assert cut.size == oracle.TILE_WORDS[fmt]
