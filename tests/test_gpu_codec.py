"""GPU parity of the block-float codec kernels against the CPU oracle — bit exact, through the C ABI."""
import json
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")
from ttmi import capi, workloads  # noqa: E402

pytestmark = pytest.mark.gpu
BFP8, BFP4 = capi.BFLOAT8_B, capi.BFLOAT4_B
HERE = os.path.dirname(os.path.abspath(__file__))
KNOWN = json.load(open(os.path.join(HERE, "golden", "reference_known_answers.json")))


def dev(a: np.ndarray):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def words_np(t) -> np.ndarray:
    return t.cpu().numpy().view(np.uint32)


def special_values(shape, seed):
    """fp32 patterns the packer treats specially: +-0, subnormals, Inf, NaN, huge and tiny exponents."""
    rng = np.random.default_rng(seed)
    n = int(np.prod(shape))
    bits = rng.integers(0, 1 << 32, size=n, dtype=np.uint64).astype(np.uint32)
    pool = np.array([0x00000000, 0x80000000, 0x00000001, 0x80000001, 0x00400000, 0x007FFFFF, 0x00800000, 0x7F800000,
                     0xFF800000, 0x7FC00000, 0xFFC00001, 0x7F7FFFFF, 0x3F7FFFFF, 0x3F800000, 0xBF800000, 0x3EFFFFFF],
                    dtype=np.uint32)
    pick = rng.random(n) < 0.5
    bits[pick] = pool[rng.integers(0, pool.size, size=int(pick.sum()))]
    # runs of 16 whose exponent fields all stay below 8 (or below 2): rows that are not fixed points of pack/unpack/pack
    tiny = np.repeat(rng.random(n // 16 + 1) < 0.3, 16)[:n]
    bits[tiny] &= np.repeat(np.where(rng.random(n // 16 + 1) < 0.5, 0x83FFFFFF, 0x80FFFFFF), 16).astype(np.uint32)[:n][tiny]
    zero_rows = rng.random(n // 16 + 1) < 0.2
    for r in np.nonzero(zero_rows)[0]:
        bits[r * 16:(r + 1) * 16] &= 0x80000000
    return bits[:n].view(np.float32).reshape(shape)


SHAPES = [(1, 1, 32, 32), (2, 3, 64, 96), (1, 1, 7, 3), (1, 2, 33, 65), (1, 1, 100, 48), (1, 1, 32, 288), (3, 1, 1, 1),
          (1, 1, 64, 4100)]


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("shape", SHAPES)
def test_from_torch_and_to_torch_paths_bit_exact(oracle, fmt, shape):
    for x in (workloads.normal_tensor(shape, seed=21), special_values(shape, seed=22)):
        want = oracle.from_torch_bfp_tiles(fmt, x)
        got = capi.pack_tensor(fmt, dev(x))
        assert np.array_equal(words_np(got), want)
        back = capi.unpack_tensor(fmt, got, shape)
        want_back = oracle.to_torch_bfp_tiles(fmt, want, shape)
        assert np.array_equal(back.cpu().numpy().view(np.uint32), want_back.view(np.uint32))
        # bf16 destination is exact: same upper halves, lower halves were zero
        back16 = capi.unpack_tensor(fmt, got, shape, dtype=torch.bfloat16)
        assert np.array_equal(back16.view(torch.int16).cpu().numpy().view(np.uint16), (want_back.view(np.uint32) >> 16).astype(np.uint16))


def rounding_boundaries(fmt, shape, seed, exponents):
    """Face rows whose shared exponent is one of `exponents` and whose elements sit on and next to the packer's rounding
    boundaries: t = m + d, d in {0, 1/2 - 2^-16, 1/2, 1/2 + 2^-16, 1 - 2^-16}, m = 0 .. 2^W, in units of the row's code step
    2^(E - 126 - W); the first element of every row is the largest code, which pins E.  All values are exact in fp32."""
    w = 7 if fmt == BFP8 else 3
    rng = np.random.default_rng(seed)
    n = int(np.prod(shape))
    rows = -(-n // 16)
    e = rng.choice(np.asarray(exponents), size=rows)
    m = rng.integers(0, (1 << w) + 1, size=(rows, 16)).astype(np.float64)
    d = rng.choice(np.array([0.0, 0.5 - 2.0 ** -16, 0.5, 0.5 + 2.0 ** -16, 1.0 - 2.0 ** -16]), size=(rows, 16))
    t = np.minimum(m + d, float((1 << w)) - 2.0 ** -16)                 # stay inside the row's binade
    t[:, 0] = float((1 << w) - 1)
    sign = rng.choice(np.array([-1.0, 1.0]), size=(rows, 16))
    x = sign * t * np.exp2(e.astype(np.float64) - 126 - w)[:, None]
    x32 = x.astype(np.float32)
    assert np.array_equal(x32.astype(np.float64), x)
    return x32.reshape(-1)[:n].reshape(shape)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("exponents", [(32, 33, 100, 127, 128, 200, 254), (31, 32, 127), (8, 20, 31, 40)])
def test_rounding_boundaries_bit_exact(oracle, fmt, exponents):
    """Ties, near-ties and code saturation in rows of every exponent range: rows the kernels take the float way (32 <= E <
    255), rows they take the integer way, and tensors where both kinds of wavefront occur."""
    shape = (1, 2, 64, 160)                                  # width 160: face rows are contiguous runs of 16 columns
    x = rounding_boundaries(fmt, shape, 24, exponents)
    want = oracle.from_torch_bfp_tiles(fmt, x)
    got = capi.pack_tensor(fmt, dev(x))
    assert np.array_equal(words_np(got), want)
    back = capi.unpack_tensor(fmt, got, shape)
    assert np.array_equal(back.cpu().numpy().view(np.uint32), oracle.to_torch_bfp_tiles(fmt, want, shape).view(np.uint32))


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_whole_block_kernel_bit_exact(oracle, fmt):
    """Tensors of at least 512 whole blocks (32 rows x 256 fp32 columns) take the straight-line pack kernel: ordinary rows by
    float arithmetic on four codes at a time, wavefronts with any other row by the integer recipe.  Special values (NaN, Inf,
    subnormals, +-0, rows that are not fixed points of pack/unpack/pack), ties / near-ties / saturation in every exponent
    range, and a source with row and batch strides; every packed word against the oracle."""
    shape = (2, 1, 1024, 2048)
    cases = [workloads.normal_tensor(shape, seed=61), special_values(shape, seed=62)]
    # mostly ordinary wavefronts with the odd element inside: -0, subnormals, the largest floats, and a NaN or Inf in a few rows
    rng = np.random.default_rng(60)
    sparse = workloads.normal_tensor(shape, seed=59).reshape(-1).view(np.uint32).copy()
    pool = np.array([0x80000000, 0x00000001, 0x807FFFFF, 0x7F7FFFFF, 0xFF7FFFFF, 0x00800000, 0x3EFFFFFF, 0x00000000], dtype=np.uint32)
    at = rng.random(sparse.size) < 0.02
    sparse[at] = pool[rng.integers(0, pool.size, size=int(at.sum()))]
    at = rng.random(sparse.size) < 1e-5
    sparse[at] = np.array([0x7F800000, 0xFFC00001], dtype=np.uint32)[rng.integers(0, 2, size=int(at.sum()))]
    cases.append(sparse.view(np.float32).reshape(shape))
    cases += [rounding_boundaries(fmt, shape, 63 + k, e) for k, e in enumerate([(32, 33, 100, 127, 128, 200, 254), (31, 32, 127), (8, 20, 31, 40)])]
    for x in cases:
        want = oracle.from_torch_bfp_tiles(fmt, x)
        assert np.array_equal(words_np(capi.pack_tensor(fmt, dev(x))), want)
    x = cases[1]
    big = np.full((2, 1024 + 3, 2048 + 64), np.float32(7.0))
    big[:, :1024, :2048] = x.reshape(2, 1024, 2048)
    d = dev(big)
    out = torch.empty(capi.lib().ttmi_tiled_size_bytes(fmt, 2, 1024, 2048) // 4, dtype=torch.int32, device="cuda")
    capi.check(capi.lib().ttmi_pack_rowmajor_as_bfp_tiles(fmt, d.data_ptr(), capi.FLOAT32, 2, 1024, 2048, 2048 + 64, (1024 + 3) * (2048 + 64), out.data_ptr(), None))
    torch.cuda.synchronize()
    assert np.array_equal(words_np(out), oracle.from_torch_bfp_tiles(fmt, x))


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_whole_block_kernel_bf16_source_bit_exact(oracle, fmt):
    """The same kernel from a bf16 source (blocks of 32 rows x 512 columns): a stress mixture and the special patterns."""
    shape = (1, 1, 4096, 2048)
    n = int(np.prod(shape))
    for x32 in (workloads.stress_mixture((1, 1, 1, n), seed=71).reshape(shape), special_values(shape, seed=72)):
        bits = (x32.view(np.uint32) >> 16).astype(np.uint16)                   # any bf16 pattern will do: truncate
        want = oracle.from_torch_bfp_tiles(fmt, workloads.bf16_bits_to_f32(bits))
        got = capi.pack_tensor(fmt, dev(bits.view(np.int16)).view(torch.bfloat16))
        assert np.array_equal(words_np(got), want)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("shape", [(1, 1, 64, 96), (2, 1, 5, 40), (1, 1, 32, 24)])
def test_bf16_source_bit_exact(oracle, fmt, shape):
    bits = workloads.f32_to_bf16_bits_rne(workloads.stress_mixture((1, 1, 1, -(-int(np.prod(shape)) // 16) * 16), seed=23).reshape(-1)[: int(np.prod(shape))]).reshape(shape)
    x32 = workloads.bf16_bits_to_f32(bits)
    want = oracle.from_torch_bfp_tiles(fmt, x32)
    got = capi.pack_tensor(fmt, dev(bits.view(np.int16)).view(torch.bfloat16))
    assert np.array_equal(words_np(got), want)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("row_major", [True, False])
@pytest.mark.parametrize("n_tiles", [1, 7, 8, 19])
def test_chunk_api_mirrors_reference_packers(oracle, fmt, row_major, n_tiles):
    x = special_values((n_tiles * 1024,), seed=30 + n_tiles)
    want = oracle.pack_fp32_vec_as_bfp_tiles(fmt, x, row_major)
    got = capi.pack_chunks(fmt, dev(x), row_major)
    assert np.array_equal(words_np(got), want)
    want_f = oracle.unpack_bfp_tiles_into_float_vec(fmt, want, row_major)
    got_f = capi.unpack_chunks(fmt, got, row_major)
    assert np.array_equal(got_f.cpu().numpy().view(np.uint32), want_f.view(np.uint32))


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_unpack_foreign_codes_every_code_and_exponent(oracle, fmt):
    """Tiles no packer would write (0x80 -> -0.0f, shift count above the exponent): every code x exponent."""
    w = 7 if fmt == BFP8 else 3
    n_codes = 2 << w
    tiles = []
    for e0 in range(0, 256, 64):
        t = np.zeros(capi.TILE_BYTES[fmt], dtype=np.uint8)
        t[:64] = np.arange(e0, e0 + 64, dtype=np.uint8)
        codes = np.arange(1024) % n_codes
        for rep in range(n_codes // 16):
            c = (np.arange(1024) + rep * 16) % n_codes
            tt = t.copy()
            if fmt == BFP8:
                tt[64:] = c.astype(np.uint8)
            else:
                tt[64:] = (c[0::2] | (c[1::2] << 4)).astype(np.uint8)
            tiles.append(tt)
        del codes
    words = np.concatenate(tiles).view(np.uint32)
    want = oracle.unpack_bfp_tiles_into_float_vec(fmt, words, False)
    got = capi.unpack_chunks(fmt, dev(words.view(np.int32)), False)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_whole_block_unpack_kernel(oracle, fmt):
    """Tensors of at least 512 whole blocks take the straight-line unpack kernel.  (a) Words the packers write for the
    special patterns: most wavefronts hold a row the integer route exists for (E < W with mantissa bits, E >= 248).
    (b) Tiles of random bytes with exponents W + 8 <= E < 248: every wavefront on the float route, with codes no packer
    writes (rows that are not normalised; sign-only codes, which come out as +0 in the to_torch sequence).  fp32 and bf16
    destinations against the oracle's to_torch sequence."""
    shapes = {torch.float32: (2, 1, 1024, 2048), torch.bfloat16: (1, 1, 4096, 2048)}
    w = 7 if fmt == BFP8 else 3
    rng = np.random.default_rng(81)
    for dtype, shape in shapes.items():
        n_tiles = int(np.prod(shape)) // 1024
        tiles = rng.integers(0, 256, size=(n_tiles, capi.TILE_BYTES[fmt]), dtype=np.uint8)
        tiles[:, :64] = rng.integers(w + 8, 248, size=(n_tiles, 64), dtype=np.uint8)
        for words in (oracle.from_torch_bfp_tiles(fmt, special_values(shape, seed=82)), tiles.reshape(-1).view(np.uint32)):
            want = oracle.to_torch_bfp_tiles(fmt, words, shape)
            got = capi.unpack_tensor(fmt, dev(words.view(np.int32)), shape, dtype=dtype)
            if dtype == torch.float32:
                assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
            else:
                assert not (want.view(np.uint32) & 0xFFFF).any()
                assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), (want.view(np.uint32) >> 16).astype(np.uint16))


def test_known_answers_on_gpu():
    for case in KNOWN["edge_single_value_rows"]["cases"]:
        row = np.zeros(1024, dtype=np.uint32)
        row[0] = int(case["bits"], 16)
        got = capi.pack_chunks(BFP8, dev(row.view(np.float32)), False)
        w = words_np(got)
        assert w[0] & 0xFF == int(case["exp"], 16) and w[16] == int(case["code"], 16), case
        back = capi.unpack_chunks(BFP8, got, False).cpu().numpy().view(np.uint32)
        assert back[0] == int(case["unpacked"], 16) and not back[1:].any(), case
    k = KNOWN["arange_tile"]
    x = np.arange(1024, dtype=np.float32)
    w8 = words_np(capi.pack_chunks(BFP8, dev(x), True))
    w4 = words_np(capi.pack_chunks(BFP4, dev(x), True))
    assert w8[0] == int(k["first_exponent_word"], 16) and w8[16] == int(k["first_mantissa_word_bfp8"], 16)
    assert w4[0] == int(k["first_exponent_word"], 16) and w4[16] == int(k["first_mantissa_word_bfp4"], 16)
    # test_bfp8_conversion.cpp:51: row-major chunk input equals tilized input
    tiled = capi.tilize(dev(x.reshape(1, 1, 32, 32)))
    assert torch.equal(capi.pack_chunks(BFP8, tiled, False).cpu(), torch.from_numpy(w8.view(np.int32)))


@pytest.mark.parametrize("dtype", [np.float32, np.uint16])
@pytest.mark.parametrize("shape", [(2, 3, 64, 96), (1, 1, 5, 40), (1, 2, 33, 65), (1, 1, 32, 1024), (1, 1, 1, 1)])
def test_tilize_untilize_match_oracle(oracle, dtype, shape):
    rng = np.random.default_rng(40)
    x = rng.integers(0, 60000, size=shape).astype(dtype)
    want = oracle.tilize_nchw_4faces(x)
    t = dev(x.view(np.int16) if dtype == np.uint16 else x)
    got = capi.tilize(t)
    assert np.array_equal(got.cpu().numpy().view(dtype), want)
    back = capi.untilize(got, shape)
    assert np.array_equal(back.cpu().numpy().view(dtype), x)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_config_roundtrip_1k_full_size(oracle, fmt):
    """fp32 [1,1,1024,1024] ~ N(0,1): the host round trip the reference runs on CPU, every packed byte compared."""
    x = workloads.roundtrip_1k()
    got = capi.pack_tensor(fmt, dev(x))
    want = oracle.from_torch_bfp_tiles(fmt, x)
    assert np.array_equal(words_np(got), want)
    back = capi.unpack_tensor(fmt, got, x.shape)
    assert np.array_equal(back.cpu().numpy().view(np.uint32), oracle.to_torch_bfp_tiles(fmt, want, x.shape).view(np.uint32))


@pytest.mark.parametrize("fmt", [BFP4, BFP8])
def test_config_stress_4k_full_size(oracle, fmt):
    """fp32 [1,1,4096,4096] mixed distribution, bit exact against the oracle, plus size-independent properties."""
    x = workloads.stress_mixture()
    d = dev(x)
    got = capi.pack_tensor(fmt, d)
    want = oracle.pack_fp32_vec_as_bfp_tiles(fmt, oracle.tilize_nchw_4faces(x), False)
    assert np.array_equal(words_np(got), want)
    back = capi.unpack_tensor(fmt, got, x.shape)
    # idempotence: pack(unpack(pack(x))) == pack(x); unpacked values fit bf16
    assert torch.equal(capi.pack_tensor(fmt, back), got)
    assert not (back.view(torch.int32) & 0xFFFF).any().item()
    want_back = oracle.untilize_nchw_4faces(oracle.unpack_bfp_tiles_into_float_vec(fmt, want, False), x.shape)
    assert np.array_equal(back.cpu().numpy().view(np.uint32), want_back.view(np.uint32))


def test_strided_source_and_empty_inputs(oracle):
    x = workloads.normal_tensor((2, 40, 80), seed=50)
    big = np.zeros((2, 48, 96), dtype=np.float32)
    big[:, :40, :80] = x
    d = dev(big)
    out = torch.empty(capi.lib().ttmi_tiled_size_bytes(BFP8, 2, 40, 80) // 4, dtype=torch.int32, device="cuda")
    capi.check(capi.lib().ttmi_pack_rowmajor_as_bfp_tiles(BFP8, d.data_ptr(), capi.FLOAT32, 2, 40, 80, 96, 48 * 96, out.data_ptr(), None))
    torch.cuda.synchronize()
    assert np.array_equal(words_np(out), oracle.from_torch_bfp_tiles(BFP8, x))
    # empty tensors are accepted and launch nothing
    assert capi.lib().ttmi_pack_rowmajor_as_bfp_tiles(BFP8, None, capi.FLOAT32, 0, 32, 32, 32, 1024, None, None) == 0
    assert capi.lib().ttmi_unpack_bfp_tiles_into_float_vec(BFP4, None, 0, 0, None, None) == 0


@pytest.mark.parametrize("fmt", [capi.BFLOAT8_B, capi.BFLOAT4_B])
def test_typecast_of_tile_ordered_tensors(oracle, fmt):
    """ttmi_typecast_tiles: block-float <-> bf16 / fp32 in tile order, one pass each way.  Towards block-float it is the host
    packers' arithmetic on the face-ordered values (bit-exact against the oracle's sequential pack); back it is exact."""
    rng = np.random.default_rng(140)
    n_tiles = 37                                                     # not a multiple of the tiles per block
    x = (rng.standard_normal(n_tiles * 1024) * np.exp2(rng.integers(-12, 12, size=n_tiles * 1024))).astype(np.float32)
    x[5000:5016] = 0.0
    x[7000] = np.float32(1e-41)
    x32 = torch.from_numpy(x).cuda()
    want = oracle.pack_fp32_vec_as_bfp_tiles(fmt, x, False)
    words = capi.typecast_tiles(x32, capi.FLOAT32, fmt)
    assert np.array_equal(words.cpu().numpy().view(np.uint32), want)
    back = oracle.unpack_bfp_tiles_into_float_vec(fmt, want, False)
    assert np.array_equal(capi.typecast_tiles(words, fmt, capi.FLOAT32).cpu().numpy().view(np.uint32), back.view(np.uint32))
    as_bf16 = capi.typecast_tiles(words, fmt, capi.BFLOAT16)
    assert as_bf16.dtype == torch.bfloat16 and np.array_equal(as_bf16.float().cpu().numpy(), back)      # at most 7 significant bits
    # from bf16 tiles: the bf16 values are packed as their exact fp32 values
    xb = x32.to(torch.bfloat16)
    assert np.array_equal(capi.typecast_tiles(xb, capi.BFLOAT16, fmt).cpu().numpy().view(np.uint32),
                          oracle.pack_fp32_vec_as_bfp_tiles(fmt, xb.float().cpu().numpy(), False))
    # bf16 <-> fp32
    assert torch.equal(capi.typecast_tiles(xb, capi.BFLOAT16, capi.FLOAT32), xb.float())
    assert torch.equal(capi.typecast_tiles(x32, capi.FLOAT32, capi.BFLOAT16), xb)                         # round to nearest even, as torch does
    with pytest.raises(RuntimeError, match="unsupported conversion"):
        capi.typecast_tiles(words, fmt, fmt)
