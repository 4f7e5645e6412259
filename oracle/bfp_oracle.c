/*
 * CPU oracle for tt-metal's block-floating-point host path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain scalar C, the
 * arithmetic of the reference host codecs so that the HIP kernels can be
 * checked bit for bit.  Nothing that ships (the C-ABI library, the ttnn /
 * tt_lib mirrors) links, loads or calls it; only tests, the smoke check and
 * the CPU-baseline leg of the benchmark do.
 *
 * Every function names the reference source it follows (paths relative to
 * the tt-metal checkout).  The structure is deliberately the reference's:
 * one thread, one face row at a time, one element at a time.
 *
 * Pinned by (see tests/test_oracle_*.py): the arange-tile words and the
 * edge-value table recorded from the compiled reference, the invariants of
 * tests/tt_metal/tt_metal/test_bfp8_conversion.cpp and
 * test_bfp4_conversion.cpp, an independent floating-point formulation of
 * the quantiser, brute force over every (exponent, shared exponent) pair and
 * every code x exponent for the unpackers, and the tilize permutation closed
 * form.  The matmul gold loop is pinned against numpy float64; pad / unpad
 * against numpy.pad and numpy slicing of the unpacked values.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdlib.h>

#define ORACLE_API __attribute__((visibility("default")))

enum { ORACLE_BFP8_B = 3, ORACLE_BFP4_B = 4 }; /* tt_eager/tensor/types.hpp:24-34 DataType values */

/* tt_metal/common/tt_backend_api_types.hpp:109-116 tile_size(): 16 exponent words + mantissa words */
static int mant_bits(int fmt) { return fmt == ORACLE_BFP8_B ? 7 : 3; }
static int words_per_tile(int fmt) { return fmt == ORACLE_BFP8_B ? 272 : 144; }

ORACLE_API uint32_t oracle_tile_size_bytes(int fmt) { return 4u * (uint32_t)words_per_tile(fmt); }

/* blockfloat_common.hpp:19-47 get_max_exp, is_exp_a == false branch:
 * largest raw biased exponent field among the 16 values of a face row. */
ORACLE_API uint32_t oracle_get_max_exp(const uint32_t *row16) {
    uint32_t best = 0;
    for (int j = 0; j < 16; ++j) {
        uint32_t e = (row16[j] & 0x7f800000u) >> 23;
        if (e > best) best = e;
    }
    return best;
}

/* bfloat8.hpp:23-87 convert_u32_to_bfp8 and blockfloat_common.hpp:67-147
 * convert_u32_to_bfp<Fmt> (is_exp_a == false, truncate_bfp_mantissa == false).
 *   +-0                       -> code 0
 *   hidden one is OR-ed in even for a zero exponent field
 *   right shift by (shared - own) truncates; shifts past 31 are done in steps
 *   then add half an output ulp, shift, saturate (no carry into the exponent)
 *   a result of zero magnitude drops its sign                              */
ORACLE_API uint32_t oracle_convert_u32_to_bfp(uint32_t bits, uint32_t shared_exp, int fmt) {
    const int w = mant_bits(fmt);
    const uint32_t drop = 24u - (uint32_t)w;       /* MANTISSA_BFP_SHIFT */
    const uint32_t top = (1u << w) - 1u;           /* MANTISSA_BFP_MAX_VAL */
    if ((bits & 0x7fffffffu) == 0) return 0;
    uint32_t frac = bits & 0x007fffffu;
    uint32_t own = (bits & 0x7f800000u) >> 23;
    uint32_t sign = bits >> 31;
    frac |= 1u << 23;
    if (shared_exp >= own) {
        uint32_t gap = shared_exp - own;
        while (gap > 31) { frac >>= 31; gap -= 31; }
        frac >>= gap;
    }
    frac += 1u << (drop - 1);
    frac >>= drop;
    if (frac > top) frac = top;
    if (frac == 0) sign = 0;
    return (sign << w) | frac;
}

/* Gather index of element j of face row (tr, tc, i) inside one 1024-element
 * tile chunk: bfloat8.hpp:128-134 / blockfloat_common.hpp:213-219. */
static inline size_t chunk_index(int row_major_chunks, int tr, int tc, int i, int j, size_t running) {
    return row_major_chunks ? (size_t)((tr * 16 + i) * 32 + tc * 16 + j) : running;
}

/* bfloat8.hpp:102-173 pack_fp32_vec_as_bfp8_tiles and
 * blockfloat_common.hpp:174-258 pack_fp32_vec_as_bfp_tiles<Bfp4_b>
 * (reached through bfloat4.hpp:23-25).
 * src: n_tiles*1024 floats, each 1024-chunk either a row-major 32x32 block
 * (row_major_input != 0) or already in 4-face order.  dst: n_tiles *
 * words_per_tile words; per tile 16 exponent words then the mantissa words,
 * faces in order (0,0) (0,1) (1,0) (1,1), element 0 in the low bits. */
ORACLE_API void oracle_pack_fp32_vec_as_bfp_tiles(int fmt, const float *src, size_t n_tiles,
                                                  int row_major_input, uint32_t *dst) {
    const int w = mant_bits(fmt);
    const int per_word = 32 / (w + 1);             /* 4 codes (bfp8) or 8 codes (bfp4) per word */
    const int wpt = words_per_tile(fmt);
    for (size_t t = 0; t < n_tiles; ++t) {
        const float *tile = src + t * 1024;
        uint32_t *exp_words = dst + t * (size_t)wpt;
        uint32_t *man_words = exp_words + 16;
        size_t running = 0, man_at = 0;
        int exp_at = 0;
        for (int tr = 0; tr < 2; ++tr)
            for (int tc = 0; tc < 2; ++tc)
                for (int i = 0; i < 16; ++i) {
                    uint32_t row[16];
                    for (int j = 0; j < 16; ++j) {
                        size_t at = chunk_index(row_major_input, tr, tc, i, j, running);
                        if (!row_major_input) ++running;
                        memcpy(&row[j], &tile[at], 4);
                    }
                    uint32_t shared = oracle_get_max_exp(row);
                    /* blockfloat_common.hpp:49-57 get_exp_dword: byte k of word w is row 4w+k */
                    if ((exp_at & 3) == 0) exp_words[exp_at >> 2] = 0;
                    exp_words[exp_at >> 2] |= (shared & 0xffu) << (8 * (exp_at & 3));
                    ++exp_at;
                    /* bfloat8.hpp:89-100 / blockfloat_common.hpp:149-172: element 0 lands in the LSBs */
                    for (int j0 = 0; j0 < 16; j0 += per_word) {
                        uint32_t word = 0;
                        for (int j = per_word - 1; j >= 0; --j) {
                            uint32_t code = oracle_convert_u32_to_bfp(row[j0 + j], shared, fmt);
                            word = (word << (w + 1)) | (code & ((1u << (w + 1)) - 1u));
                        }
                        man_words[man_at++] = word;
                    }
                }
    }
}

/* One code -> fp32 bits.  bfloat8.hpp:229-249 and bfloat4.hpp:113-146, scalar
 * form of the AVX2 lanes (is_exp_a == false):
 *   mantissa 0 -> sign bit only (0x80 / 0x8 gives -0.0f)
 *   else shift left until the top mantissa bit is set (count = sc), once
 *   more to drop it, exponent = shared - sc in int32, fields OR-ed together
 *   with 32-bit wrap when the exponent goes negative.                      */
ORACLE_API uint32_t oracle_bfp_code_to_u32(uint32_t code, uint32_t shared_exp, int fmt) {
    const int w = mant_bits(fmt);
    const uint32_t keep = (1u << w) - 1u;
    const uint32_t top_bit = 1u << (w - 1);
    uint32_t sign = (code >> w) & 1u;
    uint32_t man = code & keep;
    if (man == 0) return sign << 31;
    int32_t sc = 0;
    while (man < top_bit) { man <<= 1; ++sc; }
    man = (man << 1) & keep;
    uint32_t ex = (uint32_t)((int32_t)shared_exp - sc);
    return (sign << 31) | (ex << 23) | (man << (23 - w));
}

/* bfloat8.hpp:175-265 unpack_bfp8_tiles_into_float_vec and bfloat4.hpp:33-164
 * unpack_bfp4_tiles_into_float_vec.  row_major_output != 0 scatters each
 * tile to a row-major 32x32 block, otherwise emits 4-face order. */
ORACLE_API void oracle_unpack_bfp_tiles_into_float_vec(int fmt, const uint32_t *words, size_t n_tiles,
                                                       int row_major_output, float *dst) {
    const int w = mant_bits(fmt);
    const int per_word = 32 / (w + 1);
    const int wpt = words_per_tile(fmt);
    const int words_per_row = 16 / per_word;
    for (size_t t = 0; t < n_tiles; ++t) {
        const uint32_t *exp_words = words + t * (size_t)wpt;
        const uint32_t *man_words = exp_words + 16;
        float *tile = dst + t * 1024;
        size_t running = 0;
        for (int tr = 0; tr < 2; ++tr)
            for (int tc = 0; tc < 2; ++tc)
                for (int i = 0; i < 16; ++i) {
                    int face_row = (tr * 2 + tc) * 16 + i;
                    uint32_t shared = (exp_words[face_row >> 2] >> (8 * (face_row & 3))) & 0xffu;
                    for (int j = 0; j < 16; ++j) {
                        uint32_t word = man_words[face_row * words_per_row + j / per_word];
                        uint32_t code = (word >> ((w + 1) * (j % per_word))) & ((1u << (w + 1)) - 1u);
                        uint32_t bits = oracle_bfp_code_to_u32(code, shared, fmt);
                        size_t at = row_major_output ? (size_t)((tr * 16 + i) * 32 + tc * 16 + j) : running;
                        ++running;
                        memcpy(&tile[at], &bits, 4);
                    }
                }
    }
}

/* tt_metal/common/test_tiles.hpp:123-158 tilize_nchw followed by :24-65
 * convert_to_tile_layout, i.e. convert_layout(LIN_ROW_MAJOR -> TILED32_4FACES)
 * (:177-213), element size generic.  H and W are zero-padded up to 32. */
ORACLE_API void oracle_tilize_nchw_4faces(const void *src, uint32_t n, uint32_t c, uint32_t h, uint32_t w,
                                          uint32_t elem_size, void *dst) {
    const uint32_t hp = (h + 31u) & ~31u, wp = (w + 31u) & ~31u;
    const uint8_t *in = (const uint8_t *)src;
    uint8_t *out = (uint8_t *)dst;
    size_t linear = 0;
    for (uint32_t b = 0; b < n * c; ++b)
        for (uint32_t hs = 0; hs < hp; hs += 32)
            for (uint32_t ws = 0; ws < wp; ws += 32)
                for (uint32_t face = 0; face < 4; ++face)
                    for (uint32_t i = 0; i < 16; ++i)
                        for (uint32_t j = 0; j < 16; ++j) {
                            uint32_t r = hs + (face >> 1) * 16 + i;
                            uint32_t col = ws + (face & 1) * 16 + j;
                            uint8_t *to = out + linear * elem_size;
                            if (r < h && col < w)
                                memcpy(to, in + ((size_t)(b * h + r) * w + col) * elem_size, elem_size);
                            else
                                memset(to, 0, elem_size);
                            ++linear;
                        }
}

/* test_tiles.hpp:67-89 convert_to_flat_layout then :92-118 untilize_nchw, i.e.
 * convert_layout(TILED32_4FACES -> LIN_ROW_MAJOR).  h and w are multiples of 32. */
ORACLE_API void oracle_untilize_nchw_4faces(const void *src, uint32_t n, uint32_t c, uint32_t h, uint32_t w,
                                            uint32_t elem_size, void *dst) {
    const uint8_t *in = (const uint8_t *)src;
    uint8_t *out = (uint8_t *)dst;
    size_t linear = 0;
    for (uint32_t b = 0; b < n * c; ++b)
        for (uint32_t hs = 0; hs < h; hs += 32)
            for (uint32_t ws = 0; ws < w; ws += 32)
                for (uint32_t face = 0; face < 4; ++face)
                    for (uint32_t i = 0; i < 16; ++i)
                        for (uint32_t j = 0; j < 16; ++j) {
                            uint32_t r = hs + (face >> 1) * 16 + i;
                            uint32_t col = ws + (face & 1) * 16 + j;
                            memcpy(out + ((size_t)(b * h + r) * w + col) * elem_size, in + linear * elem_size,
                                   elem_size);
                            ++linear;
                        }
}

/* tt_metal/common/tilize_untilize.hpp:9-66 tilize(vector<bfloat16>&, m, n): the
 * second tilizer of the reference; blocks of m x n, both multiples of 32.
 * Written the way that file walks: per tile, four faces, each face row by row. */
ORACLE_API int oracle_tilize_bf16_blocks(const uint16_t *src, size_t count, uint32_t m, uint32_t n, uint16_t *dst) {
    if (count == 0 || m == 0 || n == 0 || count % ((size_t)m * n) || (m & 31) || (n & 31)) return -1;
    size_t out = 0;
    for (size_t block = 0; block < count / ((size_t)m * n); ++block) {
        const uint16_t *base = src + block * (size_t)m * n;
        for (uint32_t rt = 0; rt < m / 32; ++rt)
            for (uint32_t ct = 0; ct < n / 32; ++ct) {
                size_t corner = (size_t)rt * 32 * n + (size_t)ct * 32;
                const size_t face_start[4] = {corner, corner + 16, corner + (size_t)16 * n, corner + (size_t)16 * n + 16};
                for (int f = 0; f < 4; ++f)
                    for (uint32_t i = 0; i < 16; ++i)
                        for (uint32_t j = 0; j < 16; ++j) dst[out++] = base[face_start[f] + (size_t)i * n + j];
            }
    }
    return 0;
}

/* tilize_untilize.hpp:68-133 untilize(vector<bfloat16>&, m, n). */
ORACLE_API int oracle_untilize_bf16_blocks(const uint16_t *src, size_t count, uint32_t m, uint32_t n, uint16_t *dst) {
    if (count == 0 || m == 0 || n == 0 || count % ((size_t)m * n) || (m & 31) || (n & 31)) return -1;
    size_t out = 0;
    for (size_t block = 0; block < count / ((size_t)m * n); ++block) {
        const uint16_t *base = src + block * (size_t)m * n;
        for (uint32_t rt = 0; rt < m / 32; ++rt) {
            const uint16_t *row_of_tiles = base + (size_t)rt * 32 * n;
            for (uint32_t half = 0; half < 2; ++half)
                for (uint32_t i = 0; i < 16; ++i)
                    for (uint32_t ct = 0; ct < n / 32; ++ct) {
                        const uint16_t *tile = row_of_tiles + (size_t)ct * 1024;
                        for (uint32_t j = 0; j < 16; ++j) dst[out++] = tile[(half * 2) * 256 + i * 16 + j];
                        for (uint32_t j = 0; j < 16; ++j) dst[out++] = tile[(half * 2 + 1) * 256 + i * 16 + j];
                    }
        }
    }
    return 0;
}

/* The host sequence behind ttnn.from_torch(dtype=bfloat8_b|bfloat4_b, layout=TILE):
 *   ttnn/ttnn/operations/core.py:276-285  zero-pad H and W to multiples of 32
 *   tt_eager/tt_lib/csrc/tt_lib_bindings_tensor_pytensor.cpp:145-151  pack the padded
 *       row-major data in consecutive 1024-element chunks (row_major_input=false),
 *       declare it ROW_MAJOR
 *   tt_eager/tensor/tensor_impl.cpp:179-197 to_layout_bfloat8_b: unpack (sequential),
 *       tilize as fp32 (test_tiles.hpp convert_layout), pack again (sequential)
 * src: [batch, h, w] fp32 row-major.  dst: batch*(hp/32)*(wp/32) tiles.
 * Returns 0, or -1 when memory runs out. */
ORACLE_API int oracle_from_torch_bfp_tiles(int fmt, const float *src, uint32_t batch, uint32_t h, uint32_t w,
                                           uint32_t *dst) {
    const uint32_t hp = (h + 31u) & ~31u, wp = (w + 31u) & ~31u;
    const size_t total = (size_t)batch * hp * wp, n_tiles = total / 1024;
    float *padded = (float *)calloc(total, 4);
    float *unpacked = (float *)malloc(total * 4);
    float *tilized = (float *)malloc(total * 4);
    uint32_t *first = (uint32_t *)malloc(n_tiles * 4 * (size_t)words_per_tile(fmt));
    int rc = -1;
    if (padded && unpacked && tilized && first) {
        for (uint32_t b = 0; b < batch; ++b)
            for (uint32_t r = 0; r < h; ++r)
                memcpy(padded + ((size_t)b * hp + r) * wp, src + ((size_t)b * h + r) * w, (size_t)w * 4);
        oracle_pack_fp32_vec_as_bfp_tiles(fmt, padded, n_tiles, 0, first);
        oracle_unpack_bfp_tiles_into_float_vec(fmt, first, n_tiles, 0, unpacked);
        oracle_tilize_nchw_4faces(unpacked, 1, batch, hp, wp, 4, tilized);
        oracle_pack_fp32_vec_as_bfp_tiles(fmt, tilized, n_tiles, 0, dst);
        rc = 0;
    }
    free(padded); free(unpacked); free(tilized); free(first);
    return rc;
}

/* The host sequence behind ttnn.to_torch for a block-float tensor
 * (core.py:336-394; tensor_impl.cpp:179-197 towards ROW_MAJOR;
 * pytensor.cpp:382-393): unpack (sequential), untilize as fp32, re-pack in
 * row-major chunks, unpack again, crop the tile padding.
 * words: tiles of the padded [batch, hp, wp] tensor.  dst: [batch, h, w] fp32. */
ORACLE_API int oracle_to_torch_bfp_tiles(int fmt, const uint32_t *words, uint32_t batch, uint32_t h, uint32_t w,
                                         float *dst) {
    const uint32_t hp = (h + 31u) & ~31u, wp = (w + 31u) & ~31u;
    const size_t total = (size_t)batch * hp * wp, n_tiles = total / 1024;
    float *faces = (float *)malloc(total * 4);
    float *rows = (float *)malloc(total * 4);
    uint32_t *again = (uint32_t *)malloc(n_tiles * 4 * (size_t)words_per_tile(fmt));
    int rc = -1;
    if (faces && rows && again) {
        oracle_unpack_bfp_tiles_into_float_vec(fmt, words, n_tiles, 0, faces);
        oracle_untilize_nchw_4faces(faces, 1, batch, hp, wp, 4, rows);
        oracle_pack_fp32_vec_as_bfp_tiles(fmt, rows, n_tiles, 0, again);
        oracle_unpack_bfp_tiles_into_float_vec(fmt, again, n_tiles, 0, faces);
        for (uint32_t b = 0; b < batch; ++b)
            for (uint32_t r = 0; r < h; ++r)
                memcpy(dst + ((size_t)b * h + r) * w, faces + ((size_t)b * hp + r) * wp, (size_t)w * 4);
        rc = 0;
    }
    free(faces); free(rows); free(again);
    return rc;
}

/* tt_eager/tensor/tensor_impl.hpp:508-578 pad<T> on a 4-D row-major tensor: the output is written front to back, runs of
 * pad_value in front of and behind the input along every dimension, the input rows in between.  elem = bytes per
 * element (2 or 4); pad = the pad value already converted to the element type.  Returns -1 when the input does not fit
 * (the reference's TT_ASSERTs, :522-525). */
ORACLE_API int oracle_pad_rowmajor(const void *src, uint32_t elem, const uint32_t in_shape[4], const uint32_t out_shape[4],
                                   const uint32_t start[4], const void *pad, void *dst) {
    for (int d = 0; d < 4; ++d)
        if ((uint64_t)in_shape[d] + start[d] > out_shape[d]) return -1;
    uint32_t pad_size[4][2];
    for (int d = 0; d < 4; ++d) { pad_size[d][0] = start[d]; pad_size[d][1] = out_shape[d] - in_shape[d] - start[d]; }
    const size_t out_strides[4] = {(size_t)out_shape[1] * out_shape[2] * out_shape[3], (size_t)out_shape[2] * out_shape[3], out_shape[3], 1};
    const size_t in_strides[4] = {(size_t)in_shape[1] * in_shape[2] * in_shape[3], (size_t)in_shape[2] * in_shape[3], in_shape[3], 1};
    uint8_t *out = (uint8_t *)dst;
    const uint8_t *in = (const uint8_t *)src;
    size_t o = 0;
#define ORACLE_FILL(count) for (size_t i_ = 0; i_ < (count); ++i_) memcpy(out + (o++) * elem, pad, elem)
    ORACLE_FILL(pad_size[0][0] * out_strides[0]);
    for (uint32_t d0 = 0; d0 < in_shape[0]; ++d0) {
        ORACLE_FILL(pad_size[1][0] * out_strides[1]);
        for (uint32_t d1 = 0; d1 < in_shape[1]; ++d1) {
            ORACLE_FILL(pad_size[2][0] * out_strides[2]);
            for (uint32_t d2 = 0; d2 < in_shape[2]; ++d2) {
                ORACLE_FILL(pad_size[3][0] * out_strides[3]);
                for (uint32_t d3 = 0; d3 < in_shape[3]; ++d3) {
                    const size_t i = d3 + in_strides[2] * d2 + in_strides[1] * d1 + in_strides[0] * d0;
                    memcpy(out + (o++) * elem, in + i * elem, elem);
                }
                ORACLE_FILL(pad_size[3][1] * out_strides[3]);
            }
            ORACLE_FILL(pad_size[2][1] * out_strides[2]);
        }
        ORACLE_FILL(pad_size[1][1] * out_strides[1]);
    }
    ORACLE_FILL(pad_size[0][1] * out_strides[0]);
#undef ORACLE_FILL
    return 0;
}

/* tensor_impl.hpp:609-660 unpad<T>: the elements start..end (inclusive, every dimension) in row-major order. */
ORACLE_API int oracle_unpad_rowmajor(const void *src, uint32_t elem, const uint32_t in_shape[4], const uint32_t start[4],
                                     const uint32_t end[4], void *dst) {
    for (int d = 0; d < 4; ++d)
        if (start[d] >= in_shape[d] || end[d] >= in_shape[d] || start[d] > end[d]) return -1;
    const size_t in_strides[4] = {(size_t)in_shape[1] * in_shape[2] * in_shape[3], (size_t)in_shape[2] * in_shape[3], in_shape[3], 1};
    uint8_t *out = (uint8_t *)dst;
    const uint8_t *in = (const uint8_t *)src;
    size_t o = 0;
    for (uint32_t d0 = start[0]; d0 <= end[0]; ++d0)
        for (uint32_t d1 = start[1]; d1 <= end[1]; ++d1)
            for (uint32_t d2 = start[2]; d2 <= end[2]; ++d2)
                for (uint32_t d3 = start[3]; d3 <= end[3]; ++d3) {
                    const size_t i = d3 + in_strides[2] * d2 + in_strides[1] * d1 + in_strides[0] * d0;
                    memcpy(out + (o++) * elem, in + i * elem, elem);
                }
    return 0;
}

/* tt_eager/tensor/tensor_impl.cpp:200-215 pad_bfloat8_b (and :248-263 pad_bfloat4_b): unpack the sequential 1024-element
 * chunks to fp32, pad as a row-major fp32 tensor, pack sequentially again.  Both volumes must be whole chunks.
 * words_out: out volume / 1024 tiles.  Returns -1 on a shape error or when memory runs out. */
ORACLE_API int oracle_pad_bfp(int fmt, const uint32_t *words, const uint32_t in_shape[4], const uint32_t out_shape[4],
                              const uint32_t start[4], float pad_value, uint32_t *words_out) {
    const size_t in_vol = (size_t)in_shape[0] * in_shape[1] * in_shape[2] * in_shape[3];
    const size_t out_vol = (size_t)out_shape[0] * out_shape[1] * out_shape[2] * out_shape[3];
    if (in_vol % 1024 || out_vol % 1024) return -1;
    float *in_f = (float *)malloc(in_vol * 4 + 4), *out_f = (float *)malloc(out_vol * 4 + 4);
    int rc = -1;
    if (in_f && out_f) {
        oracle_unpack_bfp_tiles_into_float_vec(fmt, words, in_vol / 1024, 0, in_f);
        rc = oracle_pad_rowmajor(in_f, 4, in_shape, out_shape, start, &pad_value, out_f);
        if (rc == 0) oracle_pack_fp32_vec_as_bfp_tiles(fmt, out_f, out_vol / 1024, 0, words_out);
    }
    free(in_f); free(out_f);
    return rc;
}

/* tensor_impl.cpp:217-230 unpad_bfloat8_b (and :265-280 unpad_bfloat4_b): the same with unpad in the middle. */
ORACLE_API int oracle_unpad_bfp(int fmt, const uint32_t *words, const uint32_t in_shape[4], const uint32_t start[4],
                                const uint32_t end[4], uint32_t *words_out) {
    const size_t in_vol = (size_t)in_shape[0] * in_shape[1] * in_shape[2] * in_shape[3];
    size_t out_vol = 1;
    for (int d = 0; d < 4; ++d) {
        if (start[d] >= in_shape[d] || end[d] >= in_shape[d] || start[d] > end[d]) return -1;
        out_vol *= (size_t)end[d] - start[d] + 1;
    }
    if (in_vol % 1024 || out_vol % 1024) return -1;
    float *in_f = (float *)malloc(in_vol * 4 + 4), *out_f = (float *)malloc(out_vol * 4 + 4);
    int rc = -1;
    if (in_f && out_f) {
        oracle_unpack_bfp_tiles_into_float_vec(fmt, words, in_vol / 1024, 0, in_f);
        rc = oracle_unpad_rowmajor(in_f, 4, in_shape, start, end, out_f);
        if (rc == 0) oracle_pack_fp32_vec_as_bfp_tiles(fmt, out_f, out_vol / 1024, 0, words_out);
    }
    free(in_f); free(out_f);
    return rc;
}

/* tt_metal/common/bfloat16.hpp:28-38: fp32 -> bf16 keeps the upper 16 bits. */
ORACLE_API uint16_t oracle_bf16_truncate(float x) {
    uint32_t bits;
    memcpy(&bits, &x, 4);
    return (uint16_t)(bits >> 16);
}

static inline float bf16_to_float(uint16_t v) {
    uint32_t bits = (uint32_t)v << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* tests/tt_metal/tt_metal/test_gold_impls.hpp:237-290 gold_bmm (acc16 == false):
 * row-major bf16 A [nb, M, K] and B [nb, K, N], fp32 running sum in k order,
 * result left in fp32 (out_f32) and truncated to bf16 (out_bf16); either may be NULL. */
ORACLE_API void oracle_gold_bmm(const uint16_t *a, const uint16_t *b, uint32_t nb, uint32_t m, uint32_t k,
                                uint32_t n, float *out_f32, uint16_t *out_bf16) {
    for (uint32_t ib = 0; ib < nb; ++ib)
        for (uint32_t im = 0; im < m; ++im)
            for (uint32_t in = 0; in < n; ++in) {
                float acc = 0.0f;
                for (uint32_t ik = 0; ik < k; ++ik)
                    acc += bf16_to_float(a[((size_t)ib * m + im) * k + ik]) *
                           bf16_to_float(b[((size_t)ib * k + ik) * n + in]);
                size_t at = ((size_t)ib * m + im) * n + in;
                if (out_f32) out_f32[at] = acc;
                if (out_bf16) out_bf16[at] = oracle_bf16_truncate(acc);
            }
}
