"""Pins the CPU oracle's block-float codec (no GPU).

Sources of truth, none of which is the oracle's own formula retyped:
  * known answers recorded from the compiled reference (tests/golden/reference_known_answers.json);
  * the invariants of tests/tt_metal/tt_metal/test_bfp8_conversion.cpp and test_bfp4_conversion.cpp;
  * an exact-arithmetic statement of the quantiser: code = min(floor(|x| / ulp + 1/2), max), ulp =
    2**(E - 127 - (W-1)), which holds because floor((floor(y) + a) / b) == floor((y + a) / b) for
    integers a, b > 0 — the truncating pre-shift of the reference cannot change the result;
  * exact rational values of unpacked codes: sign * man * 2**(E - 127 - (W-1)).
"""
import json
import os
from fractions import Fraction

import numpy as np
import pytest

from ttmi import workloads

HERE = os.path.dirname(os.path.abspath(__file__))
KNOWN = json.load(open(os.path.join(HERE, "golden", "reference_known_answers.json")))
BFP8, BFP4 = 3, 4
W = {BFP8: 7, BFP4: 3}


def f32_bits(x):
    return np.asarray(x, dtype=np.float32).view(np.uint32)


def bits_f32(b):
    return np.asarray(b, dtype=np.uint32).view(np.float32)


def exact_value(bits: int) -> Fraction:
    """Magnitude the reference's packer *sees*: hidden one present even when the exponent field is 0."""
    e = (bits >> 23) & 0xFF
    f = bits & 0x7FFFFF
    return Fraction((1 << 23) | f) * Fraction(2) ** (e - 150)


def exact_code(bits: int, shared: int, fmt: int) -> int:
    if bits & 0x7FFFFFFF == 0:
        return 0
    w = W[fmt]
    ulp = Fraction(2) ** (shared - 127 - (w - 1))
    q = (exact_value(bits) / ulp + Fraction(1, 2)).__floor__()
    q = min(q, (1 << w) - 1)
    sign = (bits >> 31) if q else 0
    return (sign << w) | q


def test_tile_sizes(oracle):
    # tt_backend_api_types.hpp:113-116, constants.hpp:20-21
    assert oracle.lib().oracle_tile_size_bytes(BFP8) == 1088
    assert oracle.lib().oracle_tile_size_bytes(BFP4) == 576


def test_known_edge_rows_bfp8(oracle):
    for case in KNOWN["edge_single_value_rows"]["cases"]:
        bits = int(case["bits"], 16)
        row = np.zeros(1024, dtype=np.uint32)
        row[0] = bits
        words = oracle.pack_fp32_vec_as_bfp_tiles(BFP8, row.view(np.float32), False)
        assert words[0] & 0xFF == int(case["exp"], 16), case
        assert words[16] & 0xFF == int(case["code"], 16), case
        assert words[16] >> 8 == 0 and not words[17:].any()
        back = oracle.unpack_bfp_tiles_into_float_vec(BFP8, words, False).view(np.uint32)
        assert back[0] == int(case["unpacked"], 16), case
        assert not back[1:].any()


def test_known_row_with_max_one(oracle):
    k = KNOWN["row_with_max_one"]
    row = np.zeros(1024, dtype=np.float32)
    row[: len(k["values"])] = k["values"]
    words = oracle.pack_fp32_vec_as_bfp_tiles(BFP8, row, False)
    codes = [(int(words[16]) >> (8 * i)) & 0xFF for i in range(3)]
    assert codes == [int(c, 16) for c in k["codes"]]


@pytest.mark.parametrize("fmt,key", [(BFP8, "first_mantissa_word_bfp8"), (BFP4, "first_mantissa_word_bfp4")])
def test_arange_tile_known_words_and_reference_invariants(oracle, fmt, key):
    """test_bfp8_conversion.cpp:29-74 / test_bfp4_conversion.cpp:29-74 re-run on the oracle."""
    k = KNOWN["arange_tile"]
    x = np.arange(1024, dtype=np.float32)
    tiled = oracle.tilize_nchw_4faces(x.reshape(1, 1, 32, 32))
    rm_in = oracle.pack_fp32_vec_as_bfp_tiles(fmt, x, True)
    tile_in = oracle.pack_fp32_vec_as_bfp_tiles(fmt, tiled, False)
    assert rm_in[0] == int(k["first_exponent_word"], 16)
    assert rm_in[16] == int(k[key], 16)
    assert np.array_equal(rm_in, tile_in)  # :51
    rm_out = oracle.unpack_bfp_tiles_into_float_vec(fmt, rm_in, True)
    tile_out = oracle.unpack_bfp_tiles_into_float_vec(fmt, tile_in, False)
    rtol = 0.01 if fmt == BFP8 else 0.15
    # is_close(a, b, rtol, atol) of bfloat16.hpp:370-383: |a-b| <= atol + rtol*max(|a|,|b|) style bound; 8.0 dominates here
    assert np.all(np.abs(rm_out - x) <= 8.0 + rtol * np.abs(x))
    assert np.all(np.abs(tile_out - tiled) <= 8.0 + rtol * np.abs(tiled))
    assert np.array_equal(rm_out, oracle.untilize_nchw_4faces(tile_out, (1, 1, 32, 32)).reshape(-1))  # :73
    assert np.array_equal(tile_out, oracle.tilize_nchw_4faces(rm_out.reshape(1, 1, 32, 32)))  # :74


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_element_converter_every_exponent_pair_exact_arithmetic(oracle, fmt):
    """Every (own exponent, shared exponent >= own) pair with boundary mantissas, both signs."""
    w = W[fmt]
    half = 1 << (23 - w)  # half of an output ulp at gap 0, in fp32 fraction units
    fracs = sorted({0, 1, half - 1, half, half + 1, 2 * half - 1, 2 * half, 2 * half + 1, 3 * half, 0x400000,
                    0x7FFFFF - half, 0x7FFFFF - half + 1, 0x7FFFFF})
    conv = oracle.lib().oracle_convert_u32_to_bfp
    bad = 0
    for own in range(256):
        for shared in list(range(own, min(own + 30, 256))) + [255]:
            if shared < own:
                continue
            for f in fracs:
                for s in (0, 1):
                    bits = (s << 31) | (own << 23) | f
                    if conv(bits, shared, fmt) != exact_code(bits, shared, fmt):
                        bad += 1
    assert bad == 0


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_element_converter_random_exact_arithmetic(oracle, fmt):
    rng = np.random.default_rng(7)
    conv = oracle.lib().oracle_convert_u32_to_bfp
    bits = rng.integers(0, 1 << 32, size=40000, dtype=np.uint64)
    gaps = rng.integers(0, 34, size=bits.size)
    for b, g in zip(bits.tolist(), gaps.tolist()):
        own = (b >> 23) & 0xFF
        shared = min(own + g, 255)
        assert conv(b, shared, fmt) == exact_code(b, shared, fmt)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_shared_exponent_is_row_max_of_exponent_fields(oracle, fmt):
    rng = np.random.default_rng(11)
    x = rng.integers(0, 1 << 32, size=64 * 16, dtype=np.uint64).astype(np.uint32)
    words = oracle.pack_fp32_vec_as_bfp_tiles(fmt, x.view(np.float32), False)
    exps = words[:16].view(np.uint8)  # little endian: byte k of word w is row 4w+k
    want = ((x >> 23) & 0xFF).reshape(64, 16).max(axis=1)
    assert np.array_equal(exps, want.astype(np.uint8))


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_unpack_every_code_and_exponent_exact_value(oracle, fmt):
    w = W[fmt]
    dec = oracle.lib().oracle_bfp_code_to_u32
    for shared in range(256):
        for code in range(1 << (w + 1)):
            got = dec(code, shared, fmt)
            sign, man = code >> w, code & ((1 << w) - 1)
            if man == 0:
                assert got == sign << 31  # 0x80 / 0x8 -> -0.0f (bfloat8.hpp:232-244)
                continue
            sc = (w - 1) - (man.bit_length() - 1)
            if shared - sc >= 1 and shared - sc <= 254:
                val = Fraction(float(bits_f32(got)))
                assert val == (-1) ** sign * Fraction(man) * Fraction(2) ** (shared - 127 - (w - 1))
            else:
                # exponent field <= 0 or 255: release-mode behaviour of bfloat8.hpp:244-249 (no assert): the
                # int32 exponent is shifted into place with 32-bit wrap and OR-ed with sign and mantissa
                frac = ((man << (sc + 1)) & ((1 << w) - 1)) << (23 - w)
                assert got == ((sign << 31) | (((shared - sc) << 23) & 0xFFFFFFFF) | frac) & 0xFFFFFFFF


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_unpacked_values_fit_bf16_and_repack_is_identity(oracle, fmt):
    x = workloads.stress_mixture((1, 1, 64, 256), seed=5)
    words = oracle.pack_fp32_vec_as_bfp_tiles(fmt, x, False)
    vals = oracle.unpack_bfp_tiles_into_float_vec(fmt, words, False)
    assert not (vals.view(np.uint32) & 0xFFFF).any()  # at most 7 significant bits
    assert np.array_equal(oracle.pack_fp32_vec_as_bfp_tiles(fmt, vals, False), words)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_unpack_error_bound_against_input(oracle, fmt):
    """|unpack(pack(x)) - x| <= half an ulp of the row's shared exponent (plus saturation at the top code)."""
    w = W[fmt]
    x = workloads.normal_tensor((1, 1, 64, 64), seed=3)
    flat = oracle.tilize_nchw_4faces(x)
    words = oracle.pack_fp32_vec_as_bfp_tiles(fmt, flat, False)
    vals = oracle.unpack_bfp_tiles_into_float_vec(fmt, words, False)
    e = ((flat.view(np.uint32) >> 23) & 0xFF).reshape(-1, 16).max(axis=1).astype(np.int64)
    ulp = np.exp2((e - 127 - (w - 1)).astype(np.float64))
    err = np.abs(vals.astype(np.float64) - flat.astype(np.float64)).reshape(-1, 16)
    assert np.all(err <= ulp[:, None])  # half ulp rounding, one ulp where the top code saturates
    assert np.mean(err <= 0.5 * ulp[:, None]) > 0.95


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("shape", [(1, 1, 32, 32), (2, 3, 64, 96), (1, 1, 7, 3), (1, 2, 33, 65), (1, 1, 100, 48)])
def test_from_torch_sequence_equals_single_pass(oracle, fmt, shape):
    """The reference's pack(chunks) -> unpack -> tilize -> pack equals pack(tilize(pad(x))) and to_torch inverts it."""
    count = int(np.prod(shape))
    x = workloads.stress_mixture((1, 1, 1, -(-count // 16) * 16), seed=9).reshape(-1)[:count]
    x = np.ascontiguousarray(x).reshape(shape)
    full = oracle.from_torch_bfp_tiles(fmt, x)
    single = oracle.pack_fp32_vec_as_bfp_tiles(fmt, oracle.tilize_nchw_4faces(x), False)
    assert np.array_equal(full, single)
    back = oracle.to_torch_bfp_tiles(fmt, full, shape)
    hp, wp = -(-shape[2] // 32) * 32, -(-shape[3] // 32) * 32
    direct = oracle.untilize_nchw_4faces(oracle.unpack_bfp_tiles_into_float_vec(fmt, full, False), (shape[0], shape[1], hp, wp))
    assert np.array_equal(back.view(np.uint32), direct[:, :, : shape[2], : shape[3]].view(np.uint32))


def test_reference_tolerances_test_to_and_from_torch(oracle):
    """tests/ttnn/unit_tests/test_to_and_from_torch.py:22-42: 7x3 -> bfloat8_b/4_b TILE -> back."""
    rng = np.random.default_rng(0)
    x = workloads.bf16_bits_to_f32(workloads.f32_to_bf16_bits_rne(rng.random((7, 3), dtype=np.float32)))
    b8 = oracle.to_torch_bfp_tiles(BFP8, oracle.from_torch_bfp_tiles(BFP8, x), (7, 3))
    assert np.allclose(x, b8, atol=1e-2)
    b4 = oracle.to_torch_bfp_tiles(BFP4, oracle.from_torch_bfp_tiles(BFP4, x), (7, 3))
    assert np.corrcoef(x.reshape(-1), b4.reshape(-1))[0, 1] > 0.9


def test_reference_tolerances_test_tensor(oracle):
    """tests/tt_eager/python_api_testing/unit_testing/misc/test_tensor.py:26-91: (2,3,64,96), atol 1e-2 / 0.2."""
    rng = np.random.default_rng(1)
    x = rng.random((2, 3, 64, 96), dtype=np.float32)
    b8 = oracle.to_torch_bfp_tiles(BFP8, oracle.from_torch_bfp_tiles(BFP8, x), x.shape)
    b4 = oracle.to_torch_bfp_tiles(BFP4, oracle.from_torch_bfp_tiles(BFP4, x), x.shape)
    assert np.allclose(x, b8, atol=1e-2) and np.allclose(x, b4, atol=0.2)


def _special_bits(n, seed):
    rng = np.random.default_rng(seed)
    bits = rng.integers(0, 1 << 32, size=n, dtype=np.uint64).astype(np.uint32)
    pool = np.array([0, 0x80000000, 1, 0x80000001, 0x00400000, 0x007FFFFF, 0x00800000, 0x00FFFFFF, 0x01000000,
                     0x01800001, 0x02000000, 0x03000000, 0x03400000, 0x7F800000, 0x7FC00000, 0x3F800000], dtype=np.uint32)
    pick = rng.random(n) < 0.85
    bits[pick] = pool[rng.integers(0, pool.size, size=int(pick.sum()))]
    tiny = np.repeat(rng.random(-(-n // 16)) < 0.4, 16)[:n]      # runs whose exponent fields all stay below 8, or below 2
    bits[tiny] &= np.repeat(np.where(rng.random(-(-n // 16)) < 0.5, 0x83FFFFFF, 0x80FFFFFF), 16).astype(np.uint32)[:n][tiny]
    return bits


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("shape", [(1, 1, 32, 32), (1, 2, 33, 65), (1, 1, 7, 3), (2, 1, 64, 48)])
def test_from_torch_sequence_on_tiny_exponents_follows_the_zeroing_rule(oracle, fmt, shape):
    """Rows whose shared exponent is below the mantissa width are NOT fixed points of pack/unpack/pack.

    A code whose mantissa is the single bit 2**(W-1-E) unpacks to exponent field 0 with a zero fraction (bfloat8.hpp:
    240-249), i.e. to +-0, so the second pack of tt_eager/tensor/tensor_impl.cpp:179-197 writes code 0.  The full
    sequence therefore equals one pass followed by that rule — which is what the fused GPU kernel implements.
    Subnormal inputs are frequent here on purpose (zero padding makes all-tiny face rows likely)."""
    w = W[fmt]
    x = _special_bits(int(np.prod(shape)), 17).view(np.float32).reshape(shape)
    full = oracle.from_torch_bfp_tiles(fmt, x)
    single = oracle.pack_fp32_vec_as_bfp_tiles(fmt, oracle.tilize_nchw_4faces(x), False).copy()
    wpt = 272 if fmt == BFP8 else 144
    tiles = single.reshape(-1, wpt)
    exps = tiles[:, :16].copy().view(np.uint8).reshape(-1, 64).astype(np.int64)          # [tile, face row]
    per_word = 32 // (w + 1)
    shifts = (np.arange(per_word) * (w + 1)).astype(np.uint32)
    codes = (tiles[:, 16:, None] >> shifts) & ((2 << w) - 1)                       # [tile, word, slot]
    codes = codes.reshape(tiles.shape[0], 64, 16)                                  # [tile, face row, column]
    man = codes & ((1 << w) - 1)
    lone_bit = np.where(exps < w, 1 << np.clip(w - 1 - exps, 0, 31), -1)[:, :, None]
    changed = int(np.count_nonzero(man == lone_bit))
    codes = np.where(man == lone_bit, 0, codes).reshape(tiles.shape[0], -1, per_word).astype(np.uint32)
    tiles[:, 16:] = np.bitwise_or.reduce(codes << shifts, axis=2)
    assert np.array_equal(tiles.reshape(-1), full)
    assert changed > 0 or x.size < 1024  # the corner is actually exercised
    # after the sequence the data IS a fixed point: a further unpack/pack changes nothing, and to_torch's own
    # double pass equals one plain unpack
    vals = oracle.unpack_bfp_tiles_into_float_vec(fmt, full, False)
    assert np.array_equal(oracle.pack_fp32_vec_as_bfp_tiles(fmt, vals, False), full)
    hp, wp = -(-shape[2] // 32) * 32, -(-shape[3] // 32) * 32
    direct = oracle.untilize_nchw_4faces(vals, (shape[0], shape[1], hp, wp))[:, :, : shape[2], : shape[3]]
    assert np.array_equal(oracle.to_torch_bfp_tiles(fmt, full, shape).view(np.uint32), np.ascontiguousarray(direct).view(np.uint32))


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_to_torch_sequence_on_foreign_sign_only_codes(oracle, fmt):
    """Codes 0x80 / 0x8 (never written by a packer) unpack to -0.0f, but ttnn.to_torch's unpack -> pack -> unpack gives +0.0f."""
    w = W[fmt]
    words = np.zeros(272 if fmt == BFP8 else 144, dtype=np.uint32)
    words[:16] = 0x7F7F7F7F
    words[16] = (1 << w) | (0x41 << 8 if fmt == BFP8 else 0x5 << 4)
    plain = oracle.unpack_bfp_tiles_into_float_vec(fmt, words, False).view(np.uint32)
    assert plain[0] == 0x80000000
    seq = oracle.to_torch_bfp_tiles(fmt, words, (32, 32)).view(np.uint32)
    assert seq[0, 0] == 0 and seq[0, 1] == plain[1] and plain[1] != 0


def test_known_answers_follow_from_the_reference_text():
    """tests/golden/derive_known_answers.py re-derives the fixture from the reference's statements (line cited per step),
    independently of the oracle: the hidden one OR-ed into subnormals and the element-0-in-the-low-bits order are read off the
    reference's own lines there, and the fixture on file must be what that derivation gives."""
    import importlib.util

    spec = importlib.util.spec_from_file_location("derive_known_answers", os.path.join(HERE, "golden", "derive_known_answers.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert mod.strip_docs(mod.as_file(mod.derive())) == mod.strip_docs(KNOWN)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_float_route_of_the_pack_kernels_equals_the_element_converter(oracle, fmt):
    """The GPU packers compute the code of an element of an ordinary row (32 <= E < 255, elements normal or zero) as
    min(trunc(fma(|x|, 2^(126+W-E), 1/2 - 2^-25)), 2^W - 1).  The fma is one rounding (to nearest even) of the exact sum,
    which float64 holds exactly for the gaps tested here.  Mantissas on, next to and between every rounding boundary, all-ones
    mantissas and random ones, at every exponent gap; with 1/2 itself in place of 1/2 - 2^-25 one mantissa per format fails."""
    w = W[fmt]
    conv = oracle.lib().oracle_convert_u32_to_bfp
    rng = np.random.default_rng(11)
    c = float(np.float32(0.5) - np.float32(2.0 ** -25))
    failures_with_half = 0
    for gap in range(0, 26):
        own = 100
        shared = own + gap
        step = 1 << min(23, 23 - w + gap)                       # mantissa units per code step at this gap
        near = []
        for k in range(0, (1 << 24) // step + 1):
            base = k * step + step // 2                          # a tie, in units of the 24-bit mantissa
            near += [base - 2, base - 1, base, base + 1, base + 2]
        m24 = np.array(sorted({m for m in near if (1 << 23) <= m < (1 << 24)} | {(1 << 24) - 1, (1 << 24) - 2, 1 << 23}), dtype=np.int64)
        m24 = np.concatenate([m24, rng.integers(1 << 23, 1 << 24, size=2000)])
        v = m24.astype(np.float64) * 2.0 ** (w - 24 - gap)      # |x| * 2^(126+W-E), exact
        got = np.minimum(np.trunc((v + c).astype(np.float32)), (1 << w) - 1).astype(np.int64)
        half = np.minimum(np.trunc((v + 0.5).astype(np.float32)), (1 << w) - 1).astype(np.int64)
        want = np.array([conv(int((own << 23) | (m & 0x7FFFFF)), shared, fmt) for m in m24.tolist()], dtype=np.int64)
        assert np.array_equal(got, want), (gap, m24[got != want][:4])
        failures_with_half += int((half != want).sum())
    assert failures_with_half == 1
