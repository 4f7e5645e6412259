#!/usr/bin/env python3
"""Derives every entry of reference_known_answers.json from the text of the reference's host codecs, one statement at a time.

    python tests/golden/derive_known_answers.py            # prints the derivations and checks them against the JSON file
    python tests/golden/derive_known_answers.py --write    # rewrites the JSON file from the derivations

Nothing is imported from the oracle or the product.  Each function below follows one function of the reference, statement by
statement, on plain Python integers, and names the line of the reference that each statement restates (paths relative to the
tt-metal checkout).  Two conventions that the answers rest on are therefore visible in the reference's own lines, not
assumed here: the hidden one that is OR-ed into the mantissa whatever the exponent field says (bfloat8.hpp:56), and the
order of the codes inside a word, element 0 in the least significant bits (bfloat8.hpp:93-98, blockfloat_common.hpp:49-57).
"""
from __future__ import annotations

import json
import os
import struct
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
JSON_PATH = os.path.join(HERE, "reference_known_answers.json")
TRACE = []


def note(text: str) -> None:
    TRACE.append(text)


def f32_bits(x: float) -> int:
    return struct.unpack("<I", struct.pack("<f", x))[0]


def get_max_exp(row_bits) -> int:
    """tt_metal/common/blockfloat_common.hpp:19-47 get_max_exp(vec, is_exp_a = false)."""
    assert len(row_bits) == 16                              # :20  TT_ASSERT(vec.size() == 16)
    largest = 0                                             # :21  uint32_t max = 0
    for bits in row_bits:                                   # :23  for i in 0..15
        exp = (bits & 0x7F800000) >> 23                     # :25  exp = (vec[i] & 0x7f800000) >> 23
        # :27-40 is_exp_a == false on this path (tt_lib_bindings_tensor_pytensor.cpp:147): no rebias
        if exp > largest:                                   # :42
            largest = exp                                   # :43
    return largest                                          # :46


def convert_u32_to_bfp(bits: int, shared_exp: int, mant_bits: int) -> int:
    """tt_metal/common/bfloat8.hpp:23-87 convert_u32_to_bfp8 (mant_bits = 7; the shift is 17, the clamp 127), and
    tt_metal/common/blockfloat_common.hpp:67-147 convert_u32_to_bfp<Bfp4_b> (mant_bits = 3: MANTISSA_BFP_SHIFT = 21,
    MANTISSA_BFP_MAX_VAL = 7), with truncate_bfp_mantissa = false and is_exp_a = false."""
    shift = 24 - mant_bits
    top = (1 << mant_bits) - 1
    if (bits & ((1 << 31) - 1)) == 0:                       # bfloat8.hpp:26-31  +-0 -> 0
        return 0
    mantissa = bits & 0x007FFFFF                            # :33
    exp = (bits & 0x7F800000) >> 23                         # :34
    sign = (bits & 0x80000000) >> 31                        # :35
    mantissa = (1 << 23) | mantissa                         # :56  hidden one added whatever `exp` is, zero included
    if shared_exp >= exp:                                   # :58
        exp_diff = shared_exp - exp                         # :59
        while exp_diff > 31:                                # :62-65  a 32-bit value shifted by 31 at a time
            mantissa = (mantissa >> 31) & 0xFFFFFFFF
            exp_diff -= 31
        mantissa = mantissa >> exp_diff                     # :66  truncating shift
    mantissa += 1 << (shift - 1)                            # :76  "+= 1 << 16": half an ulp, i.e. ties go up in magnitude
    mantissa = mantissa >> shift                            # :77
    if mantissa > top:                                      # :78  saturate, the exponent is not touched
        mantissa = top
    if mantissa == 0:                                       # :82-84  sign only with a non-zero mantissa
        sign = 0
    return (sign << mant_bits) | mantissa                   # :85


def create_packed_as_u32(values_bits, shared_exp: int, mant_bits: int) -> int:
    """bfloat8.hpp:89-100 create_packed_bfp8_packed_as_u32 (4 codes per word) and blockfloat_common.hpp:149-172 (8 per word)."""
    per_word = 32 // (mant_bits + 1)                        # :90  nums_in_dword
    assert len(values_bits) == per_word
    word = 0                                                # :91
    mask = (1 << (32 // per_word)) - 1                      # :92
    for i in range(per_word - 1, -1, -1):                   # :93  "[0] in LSBs of dword": the last element is shifted in first
        code = convert_u32_to_bfp(values_bits[i], shared_exp, mant_bits)    # :95
        word = (word << (32 // per_word)) & 0xFFFFFFFF      # :96
        word |= code & mask                                 # :97
    return word                                             # :99


def get_exp_dword(four_exponents) -> int:
    """blockfloat_common.hpp:49-57: byte i of the word is exponent i."""
    word = 0
    for i in range(4):
        word |= (four_exponents[i] & 0xFF) << (i * 8)       # :54
    return word


def unpack_code_bfp8(code: int, shared_exp: int) -> int:
    """bfloat8.hpp:229-249, one lane of the AVX2 code written out (is_exp_a = false, so rebias_offset = 0)."""
    sign = code >> 7                                        # :229  sign = combined >> 7
    man = code & 0x7F                                       # :230
    if man == 0:                                            # :233,241,244  select_mask: a zero mantissa keeps mantissa 0 and exponent 0
        return sign << 31
    shift_cnt = 0                                           # :232
    man_shifted = man                                       # :234
    for shift_val in range(7):                              # :235-240  shift left until bit 6 is set, counting
        if man_shifted >= 0x40:
            continue
        man_shifted <<= 1
        shift_cnt = shift_val + 1
    man = (man_shifted << 1) & 0x7F                         # :241  one more shift drops the leading one
    exp = (shared_exp - shift_cnt) & 0xFFFFFFFF             # :244  _mm256_sub_epi32: wraps when shift_cnt > shared_exp (the assert of :243 is debug-only)
    return ((sign << 31) | ((exp << 23) & 0xFFFFFFFF) | (man << 16)) & 0xFFFFFFFF       # :246-249


def first_words_of_arange_tile():
    """pack_fp32_vec_as_bfp8_tiles (bfloat8.hpp:102-173) and pack_fp32_vec_as_bfp_tiles<Bfp4_b> (blockfloat_common.hpp:174-258)
    with row_major_input = true on the tile 0, 1, ..., 1023 of tests/tt_metal/tt_metal/test_bfp8_conversion.cpp:29-32: only
    the first exponent word (rows 0..3 of face 0) and the first mantissa word (row 0, columns 0..) are derived."""
    exponents = []
    first = {}
    for i in range(4):                                      # :127  rows i of sub-tile (tr, tc) = (0, 0), :125-126
        row = []
        for j in range(16):                                 # :130
            data_index = (0 * 16 + i) * 32 + (0 * 16 + j)   # :132  row_major_input: (tr*16 + i)*32 + (tc*16 + j)
            row.append(f32_bits(float(data_index)))         # :136-138
        exp = get_max_exp(row)                              # :141
        exponents.append(exp)                               # :142
        note(f"arange tile, face 0 row {i}: values {i * 32}..{i * 32 + 15}, shared exponent 0x{exp:02x}")
        if i == 0:
            first["bfp8"] = create_packed_as_u32(row[0:4], exp, 7)          # :150-155  every 4 values one word
            first["bfp4"] = create_packed_as_u32(row[0:8], exp, 3)          # blockfloat_common.hpp:230-236  every 8 values
    return get_exp_dword(exponents), first["bfp8"], first["bfp4"]           # :144-147


def derive() -> dict:
    edge = []
    for bits in (0x00000001, 0x00400000, 0x00800000, 0x80000000, 0x7F800000, 0x7FC00000, 0x3F7FFFFF):
        row = [bits] + [0] * 15                             # one value in an otherwise all-zero face row
        exp = get_max_exp(row)
        code = convert_u32_to_bfp(bits, exp, 7)
        back = unpack_code_bfp8(code, exp)
        note(f"single value 0x{bits:08x}: shared exponent 0x{exp:02x}, code 0x{code:02x}, unpacks to 0x{back:08x}")
        edge.append({"bits": f"0x{bits:08x}", "exp": f"0x{exp:02x}", "code": f"0x{code:02x}", "unpacked": f"0x{back:08x}"})
    values = [1.0, 0.0077, -1e-10]
    row = [f32_bits(v) for v in values] + [0] * 13
    exp = get_max_exp(row)
    codes = [convert_u32_to_bfp(b, exp, 7) for b in row[:3]]
    note(f"row with maximum 1.0: shared exponent 0x{exp:02x}, codes {[hex(c) for c in codes]}")
    exp_word, word8, word4 = first_words_of_arange_tile()
    note(f"arange tile: exponent word 0x{exp_word:08x}, first mantissa word bfp8 0x{word8:08x}, bfp4 0x{word4:08x}")
    return {
        "edge_single_value_rows": edge,
        "row_with_max_one": {"values": values, "codes": [f"0x{c:02x}" for c in codes]},
        "arange_tile": {"first_exponent_word": f"0x{exp_word:08x}", "first_mantissa_word_bfp8": f"0x{word8:08x}",
                        "first_mantissa_word_bfp4": f"0x{word4:08x}"},
    }


def as_file(derived: dict) -> dict:
    return {
        "_provenance": "Derived by tests/golden/derive_known_answers.py from the text of the reference's host codecs "
                       "(tt_metal/common/bfloat8.hpp, blockfloat_common.hpp), statement by statement with the line cited per "
                       "step; first recorded from a build of those headers while the reference was surveyed, and identical to it.",
        "edge_single_value_rows": {
            "_doc": "one fp32 value (bits) in an otherwise all-zero face row, BFP8_B: shared exponent byte, code byte, unpacked fp32 bits",
            "cases": derived["edge_single_value_rows"]},
        "row_with_max_one": dict(
            _doc="BFP8_B, face row whose largest value is 1.0: values below half an ulp of the shared exponent pack to code 0x00 (sign dropped)",
            **derived["row_with_max_one"]),
        "arange_tile": dict(
            _doc="fp32 tile holding 0..1023 in row-major order (tests/tt_metal/tt_metal/test_bfp8_conversion.cpp:29-32): first exponent "
                 "word and first mantissa word of the packed tile",
            **derived["arange_tile"]),
    }


def strip_docs(node):
    if isinstance(node, dict):
        return {k: strip_docs(v) for k, v in node.items() if not k.startswith("_")}
    if isinstance(node, list):
        return [strip_docs(v) for v in node]
    return node


def main() -> int:
    derived = as_file(derive())
    if "--write" in sys.argv:
        with open(JSON_PATH, "w") as f:
            json.dump(derived, f, indent=1)
            f.write("\n")
        print(f"wrote {JSON_PATH}")
        return 0
    for line in TRACE:
        print(line)
    on_file = json.load(open(JSON_PATH))
    same = strip_docs(on_file) == strip_docs(derived)
    print("matches" if same else "DIFFERS FROM", JSON_PATH)
    return 0 if same else 1


if __name__ == "__main__":
    sys.exit(main())
