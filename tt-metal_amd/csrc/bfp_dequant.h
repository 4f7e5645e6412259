// Device-side pieces shared by the block-float GEMM kernels: operand types, the LDS layout of staged packed tiles,
// and the exact expansion of block-float codes into bf16 MFMA operands.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ttmi.h"

namespace ttmi {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // first-class 16-byte value: stays in registers

// LDS stage of one wavefront = the 2 adjacent packed tiles of one unit, placed by direct global->LDS loads
// (global_load_lds_dwordx4: lane l of load i writes its 16 bytes at stage + i*1024 + l*16, from any global
// address it likes).  Slots are laid out so that what one ds_read touches sits in different banks:
//   face (tile t, face f = 2h + fc) has index h*4 + t*2 + fc and starts at index * face_stride, i.e. every face is
//   followed by one 16-byte pad slot; the 8 exponent chunks follow the faces; the remaining slots are dummies.
template <int W> struct Wfmt;
template <> struct Wfmt<7> {
    static constexpr int tile_bytes = 1088, chunks = 68, row_bytes = 16;
    static constexpr int face_slots = 17, face_stride = face_slots * 16;   // 16 rows + 1 pad
    static constexpr int exp_base = 8 * face_stride;                        // 2176
    static constexpr int loads = 3, stage_bytes = loads * 1024;
    static constexpr int bias_exp = 133;                                    // value = mantissa * 2^(E - 133)
    static constexpr float unscale = 1.0f / 64.0f;                          // 2^(127 - bias_exp)
};
template <> struct Wfmt<3> {
    static constexpr int tile_bytes = 576, chunks = 36, row_bytes = 8;
    static constexpr int face_slots = 9, face_stride = face_slots * 16;    // 8 chunks of 2 rows + 1 pad
    static constexpr int exp_base = 8 * face_stride;                        // 1152
    static constexpr int loads = 2, stage_bytes = loads * 1024;
    static constexpr int bias_exp = 129;                                    // value = mantissa * 2^(E - 129)
    static constexpr float unscale = 1.0f / 4.0f;                           // 2^(127 - bias_exp)
};

// LDS stage of one wavefront of the 128-column kernel = the 4 adjacent packed tiles of one unit, brought in by direct
// global->LDS loads in which four neighbouring lanes always fetch one aligned 64-byte piece of memory ("quad": 4 face rows
// of BFP8, 8 of BFP4).  That is what the address coalescing of the vector memory pipe wants; with a pad slot per face, as
// Wfmt has it, every piece is split over two groups of four lanes, and the loads, not the memory, bound the kernel
// (measured on the Falcon h_to_4h shape without arithmetic: 17.4 us against 15.4 us).  What one ds_read touches still
// lies in 64 different banks, because a quad may go to any quad position of its load and every load may start at any
// multiple of 16 bytes:
//   tile t (0..3) has a load of its own that starts 16 t (BFP4: 48 t) bytes off a multiple of 64, so tiles differ in the
//         16-byte phase;
//   BFP8  the 16 quads of a tile's faces (memory order: face f = 2s + fc, row group kh, row quad rq) are placed at
//         position 8s + 4rq + 2kh + fc: one pass of a ds_read2_b32 (s, rq and the row inside the quad are common to all
//         lanes) finds the four (kh, fc) of a tile in four different 64-byte phases, fc in the lowest.  The exponents of
//         the four tiles come with a fifth load (16 lanes).
//   BFP4  a tile is 9 quads: the exponents, then the quad of (face 2s + fc, row group kh) at position 1 + 4s + 2kh + fc.
// With fc in the lowest position bit the 32 lanes of a half wavefront (kh is the upper half) already differ modulo 128
// bytes: the counters say that a ds_read2_b32 is served half a wavefront at a time from 32 banks (a layout that was
// conflict-free only modulo 256 bytes read 4 conflict cycles per instruction).
template <int W> struct WideFmt;
template <> struct WideFmt<7> {
    static constexpr int tile_bytes = 1088, chunks = 68, row_bytes = 16;
    static constexpr int loads = 5;                                    // 4 tiles' faces + the exponents
    static constexpr int load_stride = 1024 + 16;
    static constexpr int exp_base = 4 * load_stride, unit_bytes = exp_base + 1024;
    static constexpr int slab_bytes = 512;                             // mantissas of slab 1 lie this far behind slab 0
    // byte offsets of the four ds_read2_b32 of a slab (rows 2i and 2i + 1) from the lane's address
    static constexpr int pair_offset(int i) { return (i >> 1) * 256 + (i & 1) * 32; }
    static constexpr int row_step = 16;
};
template <> struct WideFmt<3> {
    static constexpr int tile_bytes = 576, chunks = 36, row_bytes = 8;
    static constexpr int loads = 4;                                    // one per tile: 36 of the 64 lanes fetch
    static constexpr int load_stride = 1024 + 48;                      // 48 t mod 64 = 0, 48, 32, 16
    static constexpr int exp_base = 0, unit_bytes = 4 * load_stride;
    static constexpr int slab_bytes = 256;
    static constexpr int pair_offset(int i) { return i * 16; }
    static constexpr int row_step = 8;
};
// chunk (16 bytes, counted from the start of the unit's 4 tiles) that this lane fetches in load l of a unit
template <int W> __host__ __device__ __forceinline__ void wide_stage_chunks(int lane, uint32_t (&chunk_of)[WideFmt<W>::loads]) {
    using F = WideFmt<W>;
#pragma unroll
    for (int l = 0; l < F::loads; ++l) {
        uint32_t c;
        if (W == 7 && l < 4) {
            const uint32_t pos = lane >> 2, s = pos >> 3, rq = (pos >> 2) & 1, kh = (pos >> 1) & 1, fc = pos & 1;
            c = l * F::chunks + 4 + 4 * (8 * s + 4 * fc + 2 * kh + rq) + (lane & 3);   // the memory quad that belongs at this position
        } else if (W == 7) {
            const uint32_t e = lane < 15 ? (uint32_t)lane : 15u;        // idle lanes repeat the last chunk
            c = (e >> 2) * F::chunks + (e & 3);
        } else {
            const uint32_t slot = lane < F::chunks - 1 ? (uint32_t)lane : (uint32_t)F::chunks - 1;      // idle lanes repeat the last chunk
            uint32_t quad = slot >> 2;
            if (quad >= 1) { const uint32_t p = quad - 1, s = p >> 2, kh = (p >> 1) & 1, fc = p & 1; quad = 1 + 4 * s + 2 * fc + kh; }
            c = l * F::chunks + 4 * quad + (slot & 3);
        }
        chunk_of[l] = c;
    }
}
// this lane's LDS byte offsets inside a stage for slab 0: exponents (8 bytes: k rows 8kh .. 8kh + 7 of its face) and
// mantissa word of k row 8kh (lane: tile t, face column fc, word q, row group kh)
template <int W> __host__ __device__ __forceinline__ uint32_t wide_exp_at(int t, int fc, int kh) {
    using F = WideFmt<W>;
    return (W == 7 ? F::exp_base + t * 64 : t * F::load_stride) + fc * 16 + kh * 8;
}
template <int W> __host__ __device__ __forceinline__ uint32_t wide_mant_at(int t, int fc, int q, int kh) {
    using F = WideFmt<W>;
    return W == 7 ? t * F::load_stride + (2 * kh + fc) * 64 + q * 4 : t * F::load_stride + 64 + (2 * kh + fc) * 64 + (q >> 1) * 4;
}

// s_waitcnt vmcnt(n) only (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14)
template <int N> __device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 0xf) | (0x7 << 4) | (0xf << 8) | ((N >> 4) << 14));
    asm volatile("" ::: "memory");
}

// Scale of a face row from its shared exponent byte: the byte moved into the exponent field of a float, 2^(E - 127) —
// 2^(bias_exp - 127) times too large for every row alike (whoever stores the sums takes that power of two out again,
// exactly).  E = 0 is read as E = 1, the IEEE convention for a zero exponent field, which is also what the hidden-one
// form of the streaming kernels gives: every GEMM kernel treats such rows (fp32 subnormal sources) alike.
__device__ __forceinline__ float row_scale(uint32_t e) { return __uint_as_float(max(e, 1u) << 23); }

template <int ACT> __device__ __forceinline__ float apply_activation(float x) {
    if (ACT == TTMI_ACT_RELU) return x > 0.f ? x : 0.f;
    if (ACT == TTMI_ACT_GELU) return 0.5f * x * (1.f + erff(x * 0.70710678118654752440f));
    if (ACT == TTMI_ACT_SILU) return x / (1.f + __expf(-x));
    return x;
}

// two floats -> two bf16 in one word (lo in the low half), round to nearest even: one v_cvt_pk_bf16_f32 on gfx950
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_rne(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// v_cvt_f32_ubyteN: byte N of a word as float, one instruction (the compiler otherwise extracts the field first)
template <int SEL> __device__ __forceinline__ float byte_to_float(uint32_t word) {
    float r;
    if (SEL == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(word));
    else if (SEL == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(word));
    else if (SEL == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(word));
    else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(word));
    return r;
}

// Eight weights of one output column, k rows 8g..8g+7, as the bf16 B operand of an MFMA.
//   words[jj]  mantissa word of k row 8g+jj that contains this column's code, sign bit at bit 7 of its byte
//   mags[jj]   the same word with only the mantissas left, one per byte
//   scale[jj]  2^(E - bias_exp) of that row
//   SEL        which byte of the word
// Per pair of rows: 2 x v_cvt_f32_ubyteN, 2 x v_mul_f32, v_perm_b32 (keep the upper halves = exact bf16),
// v_perm_b32 (fetch the two sign bytes) and v_and_or_b32.
template <int SEL>
__device__ __forceinline__ bf16x8 weights_operand8(const uint32_t (&words)[8], const uint32_t (&mags)[8], const float (&scale)[8]) {
    uint32_t packed[4];
    constexpr uint32_t sign_sel = ((4u + SEL) << 24) | (0x0cu << 16) | ((uint32_t)SEL << 8) | 0x0cu;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t v0 = __float_as_uint(byte_to_float<SEL>(mags[2 * p]) * scale[2 * p]);
        const uint32_t v1 = __float_as_uint(byte_to_float<SEL>(mags[2 * p + 1]) * scale[2 * p + 1]);
        const uint32_t both = __builtin_amdgcn_perm(v1, v0, 0x07060302u);
        const uint32_t signs = __builtin_amdgcn_perm(words[2 * p + 1], words[2 * p], sign_sel);
        packed[p] = (signs & 0x80008000u) | both;
    }
    return __builtin_bit_cast(bf16x8, make_uint4(packed[0], packed[1], packed[2], packed[3]));
}

// Eight BFLOAT8_B activations of one face row (codes in `w0`, `w1` in memory order, shared exponent byte `e`) as the bf16 A
// operand of an MFMA, 64 times too large: mantissa x 2^(max(E, 1) - 127), exact (a 7-bit mantissa fits a bf16), where the
// reference unpacker gives mantissa x 2^(E - 127 - 6) (bfloat8.hpp:229-249).  Whoever stores the sums takes the 64 out.
template <int LO> __device__ __forceinline__ uint32_t activations_pair(uint32_t w, uint32_t mags, float scale) {
    const uint32_t v0 = __float_as_uint(byte_to_float<LO>(mags) * scale);
    const uint32_t v1 = __float_as_uint(byte_to_float<LO + 1>(mags) * scale);
    const uint32_t both = __builtin_amdgcn_perm(v1, v0, 0x07060302u);                         // the upper halves: exact bf16
    constexpr uint32_t sign_sel = ((uint32_t)(LO + 1) << 24) | (0x0cu << 16) | ((uint32_t)LO << 8) | 0x0cu;
    return (__builtin_amdgcn_perm(w, w, sign_sel) & 0x80008000u) | both;
}
__device__ __forceinline__ u32x4 activations_operand8(uint32_t w0, uint32_t w1, uint32_t e) {
    const float scale = row_scale(e & 0xffu);
    const uint32_t m0 = w0 & 0x7f7f7f7fu, m1 = w1 & 0x7f7f7f7fu;
    u32x4 out;
    out[0] = activations_pair<0>(w0, m0, scale);
    out[1] = activations_pair<2>(w0, m0, scale);
    out[2] = activations_pair<0>(w1, m1, scale);
    out[3] = activations_pair<2>(w1, m1, scale);
    return out;
}

// Fills `chunk_of[l]` with the global chunk (16 bytes, counted from the start of a 2-tile run) that lands in this
// lane's slot of direct-to-LDS load l, for the stage layout described at Wfmt.
template <int W> __device__ __forceinline__ void stage_chunks(int lane, uint32_t (&chunk_of)[Wfmt<W>::loads]) {
    using F = Wfmt<W>;
#pragma unroll
    for (int l = 0; l < F::loads; ++l) {
        const uint32_t slot = l * 64 + lane;
        const uint32_t face_idx = slot / F::face_slots, within = slot % F::face_slots;
        uint32_t chunk = 0;                                               // pads and dummies refetch chunk 0
        if (face_idx < 8) {
            if (within < (uint32_t)F::face_slots - 1) {
                const uint32_t h = face_idx >> 2, t = (face_idx >> 1) & 1, f = 2 * h + (face_idx & 1);
                chunk = t * F::chunks + 4 + f * (F::face_slots - 1) + within;
            }
        } else if (slot - 8 * F::face_slots < 8) {
            const uint32_t e = slot - 8 * F::face_slots;                  // exponent chunk e%4 of tile e/4
            chunk = (e >> 2) * F::chunks + (e & 3);
        }
        chunk_of[l] = chunk;
    }
}

// What one lane reads from LDS for 8 k rows of one face of a staged pair of packed tiles (8 exponent bytes, 8 mantissa
// words; exp_at / mant_at: this lane's LDS byte addresses in stage 0, see Wfmt).  LDS reads are written as inline
// assembly: the compiler orders every LDS read it knows of behind ALL outstanding direct-to-LDS loads (it cannot tell
// that they write other stages), which would drain the prefetch pipeline at every unit.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
struct SlabRaw { u32x2 e01, w01, w23, w45, w67; };

// requested here (EXP_OFF / MANT_OFF are compile-time byte offsets; the caller waits with wait_slab / wait_slabs, which
// carry the results as operands so that nothing that uses them can be scheduled in front of the wait)
template <int W, int EXP_OFF, int MANT_OFF> __device__ __forceinline__ void slab_read(uint32_t exp_at, uint32_t mant_at, SlabRaw &r) {
    constexpr int R = Wfmt<W>::row_bytes / 4;
    const uint32_t mant = mant_at + MANT_OFF;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(r.e01) : "v"(exp_at), "n"(EXP_OFF));
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(r.w01) : "v"(mant), "n"(0 * R), "n"(1 * R));
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(r.w23) : "v"(mant), "n"(2 * R), "n"(3 * R));
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(r.w45) : "v"(mant), "n"(4 * R), "n"(5 * R));
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(r.w67) : "v"(mant), "n"(6 * R), "n"(7 * R));
}
// the same for a stage laid out as WideFmt describes
template <int W, int EXP_OFF, int MANT_OFF> __device__ __forceinline__ void wide_slab_read(uint32_t exp_at, uint32_t mant_at, SlabRaw &r) {
    using F = WideFmt<W>;
    constexpr int R = F::row_step / 4;
    const uint32_t mant = mant_at + MANT_OFF;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(r.e01) : "v"(exp_at), "n"(EXP_OFF));
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(r.w01) : "v"(mant), "n"(F::pair_offset(0) / 4), "n"(F::pair_offset(0) / 4 + R));
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(r.w23) : "v"(mant), "n"(F::pair_offset(1) / 4), "n"(F::pair_offset(1) / 4 + R));
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(r.w45) : "v"(mant), "n"(F::pair_offset(2) / 4), "n"(F::pair_offset(2) / 4 + R));
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(r.w67) : "v"(mant), "n"(F::pair_offset(3) / 4), "n"(F::pair_offset(3) / 4 + R));
}
__device__ __forceinline__ void wait_slab(SlabRaw &a) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a.e01), "+v"(a.w01), "+v"(a.w23), "+v"(a.w45), "+v"(a.w67)::"memory");
}
__device__ __forceinline__ void wait_slabs(SlabRaw &a, SlabRaw &b) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a.e01), "+v"(a.w01), "+v"(a.w23), "+v"(a.w45), "+v"(a.w67),
                                          "+v"(b.e01), "+v"(b.w01), "+v"(b.w23), "+v"(b.w45), "+v"(b.w67)::"memory");
}
// BFLOAT4_B: exact expansion into single operands through the scaled fp8-to-bf16 conversion.  A 3-bit mantissa 0..7 is an
// e4m3 value (bytes 00 38 40 44 48 4A 4C 4E), and v_cvt_scalef32_pk_bf16_fp8 turns two of them into bf16 values times a power
// of two, here 2^(max(E, 1) - 127): the operand holds mantissa x 2^(max(E, 1) - 127) = 4 x the weight (Wfmt<3>::unscale takes
// the 4 out of the sums), exactly.  About 2.75 vector-ALU instructions per weight, and one matrix instruction per operand
// where the hidden-one form below needs two, and the sums see nothing but products with the weights.  Edge rows as in the
// tiled kernels: E = 0 is read as E = 1; E = 254 overflows
// for mantissas >= 2; E = 255 makes the 16 columns that share the exponent non-finite.
__device__ __forceinline__ void slab_expand_bfp4(const SlabRaw &r, int q, bf16x8 (&bop)[4]) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const uint32_t words[8] = {r.w01[0], r.w01[1], r.w23[0], r.w23[1], r.w45[0], r.w45[1], r.w67[0], r.w67[1]};
    uint32_t lo[8], hi[8];         // (columns 0, 1) and (columns 2, 3) of row jj as bf16 pairs
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
        const uint32_t e = (r.e01[jj >> 2] >> (8 * (jj & 3))) & 0xffu;
        const float scale = __uint_as_float((e > 1u ? e : 1u) << 23);
        uint32_t v = (words[jj] >> (16 * (q & 1))) & 0xffffu;
        v = (v | (v << 8)) & 0x00ff00ffu;
        v = (v | (v << 4)) & 0x0f0f0f0fu;                                   // one code per byte
        const uint32_t fp8 = ((v << 4) & 0x80808080u) | __builtin_amdgcn_perm(0x4E4C4A48u, 0x44403800u, v & 0x07070707u);
        lo[jj] = __builtin_bit_cast(uint32_t, (bf16x2_t)__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(fp8, scale, false));
        hi[jj] = __builtin_bit_cast(uint32_t, (bf16x2_t)__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(fp8, scale, true));
    }
    uint32_t packed[4][4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        packed[0][p] = __builtin_amdgcn_perm(lo[2 * p + 1], lo[2 * p], 0x05040100u);
        packed[1][p] = __builtin_amdgcn_perm(lo[2 * p + 1], lo[2 * p], 0x07060302u);
        packed[2][p] = __builtin_amdgcn_perm(hi[2 * p + 1], hi[2 * p], 0x05040100u);
        packed[3][p] = __builtin_amdgcn_perm(hi[2 * p + 1], hi[2 * p], 0x07060302u);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) bop[j] = __builtin_bit_cast(bf16x8, make_uint4(packed[j][0], packed[j][1], packed[j][2], packed[j][3]));
}

// Which form the 128-column kernel feeds the matrix cores: single exact operands where a workgroup multiplies the weights
// with two 32-row bands (the expansion is shared by the bands and the matrix instructions are what such a launch waits for:
// BFLOAT4_B 22.0 against 23.6 us for [64, 4096] x [4096, 14336], BFLOAT8_B 32.0 against 33.3 us for [64, 4544] x
// [4544, 18176]); the hidden-one form below with one band (BFLOAT4_B 14.5 against 15.3 us for [32, 4096] x [4096, 14336];
// BFLOAT8_B 23.1 against 24.9 us for the Falcon shape).
template <int W, int BANDS> constexpr bool single_operand() { return BANDS == 2; }
// BFLOAT8_B the same way: convert, multiply by the row's power of two, keep the upper halves (weights_operand8)
__device__ __forceinline__ void slab_expand_bfp8(const SlabRaw &r, bf16x8 (&bop)[4]) {
    const uint32_t words[8] = {r.w01[0], r.w01[1], r.w23[0], r.w23[1], r.w45[0], r.w45[1], r.w67[0], r.w67[1]};
    float scale[8];
    uint32_t mags[8];
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) { scale[jj] = row_scale((r.e01[jj >> 2] >> (8 * (jj & 3))) & 0xffu); mags[jj] = words[jj] & 0x7f7f7f7fu; }
    bop[0] = weights_operand8<0>(words, mags, scale);
    bop[1] = weights_operand8<1>(words, mags, scale);
    bop[2] = weights_operand8<2>(words, mags, scale);
    bop[3] = weights_operand8<3>(words, mags, scale);
}

// Expansion without arithmetic ("hidden-one form"), for kernels that are bound by vector-ALU issue rather than by the
// matrix pipe.  A code (sign s, mantissa m of W bits) under the shared exponent E of its face row is written into a bf16 as
//      hi[15] = s, hi[14:7] = E, hi[6:7-W] = m          value  +-(1 + m / 2^W) * 2^(E - 127)
// and a second operand carries sign and exponent alone
//      lo[15] = s, lo[14:7] = E                          value  +-2^(E - 127)
// so that hi - lo = +-m * 2^(E - 127 - W), half of the weight m * 2^(E - 127 - (W - 1)) the reference unpacker produces
// (bfloat8.hpp:229-249, bfloat4.hpp:113-146): A.W = hidden_unscale * (A.hi - A.lo), exactly (both operands and every
// product are exact; only the fp32 additions see other intermediate sums than a product with the expanded weight would).
// Nothing is converted, multiplied or normalised: per pair of k rows one v_perm_b32 brings the two codes of a column
// together and two v_and_or_b32 assemble hi and lo; the exponent field of a pair of rows is prepared once for the four
// operands.  Edge rows: E = 0 makes hi a bf16 subnormal and lo a zero, and the matrix cores keep subnormals, so such a row
// is read with the scale of E = 1 (the IEEE convention for a zero exponent field; all-zero rows give exactly 0);
// E = 255 (Inf / NaN sources) makes the sums of the 16 columns that share the exponent non-finite; every other exponent,
// 254 included, is exact.
constexpr float hidden_unscale = 2.0f;
// what the sums of a streaming kernel are multiplied by
template <int W, int BANDS> constexpr float decode_unscale() { return single_operand<W, BANDS>() ? Wfmt<W>::unscale : hidden_unscale; }

// exponent field of k rows (2p, 2p + 1), one in each half of a word
__device__ __forceinline__ uint32_t hidden_pair_field(const u32x2 e01, int p) {
    const uint32_t ew = e01[p >> 1];
    const uint32_t spread = (p & 1) ? __builtin_amdgcn_perm(0u, ew, 0x0c030c02u) : __builtin_amdgcn_perm(0u, ew, 0x0c010c00u);   // [E(2p), 0, E(2p+1), 0]
    return spread << 7;
}

template <int W> __device__ __forceinline__ void slab_expand_hidden(const SlabRaw &r, int q, bf16x8 (&hi)[4], bf16x8 (&lo)[4]) {
    const uint32_t words[8] = {r.w01[0], r.w01[1], r.w23[0], r.w23[1], r.w45[0], r.w45[1], r.w67[0], r.w67[1]};
    uint32_t hi_w[4][4], lo_w[4][4];     // [operand j][row pair p]
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t field = hidden_pair_field(r.e01, p);
        if constexpr (W == 7) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // both codes of column j, each in both bytes of its half
                const uint32_t sel = ((4u + j) << 24) | ((4u + j) << 16) | ((uint32_t)j << 8) | (uint32_t)j;
                const uint32_t both = __builtin_amdgcn_perm(words[2 * p + 1], words[2 * p], sel);
                hi_w[j][p] = (both & 0x807f807fu) | field;
                lo_w[j][p] = (both & 0x80008000u) | field;
            }
        } else {
            // this lane's four codes of each row: the 16-bit half (q & 1) of the row's word, row 2p in the low half
            const uint32_t both = __builtin_amdgcn_perm(words[2 * p + 1], words[2 * p], (q & 1) ? 0x07060302u : 0x05040100u);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // code j sits at bits 4j..4j+3 of each half: its sign goes to bit 15, its mantissa to bits 6..4 (bits that a
                // shift carries over from the other half never reach the masked positions)
                const uint32_t s_at = j == 3 ? both : both << (12 - 4 * j);
                const uint32_t m_at = j == 0 ? both << 4 : j == 1 ? both : both >> (4 * j - 4);
                lo_w[j][p] = (s_at & 0x80008000u) | field;
                hi_w[j][p] = (m_at & 0x00700070u) | lo_w[j][p];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        hi[j] = __builtin_bit_cast(bf16x8, make_uint4(hi_w[j][0], hi_w[j][1], hi_w[j][2], hi_w[j][3]));
        lo[j] = __builtin_bit_cast(bf16x8, make_uint4(lo_w[j][0], lo_w[j][1], lo_w[j][2], lo_w[j][3]));
    }
}

// ---- the packer's arithmetic for one element and one face row (used by the codec kernels and by GEMM epilogues that
// write block-float output) -------------------------------------------------------------------------------------------
// max over the 2 or 4 lanes that share a face row (lanes are aligned quads / pairs)
template <int LPR> __device__ __forceinline__ uint32_t row_max(uint32_t v) {
    uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1 /* quad_perm:[1,0,3,2] */, 0xf, 0xf, true);
    v = v > o ? v : o;
    if (LPR == 4) {
        o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E /* quad_perm:[2,3,0,1] */, 0xf, 0xf, true);
        v = v > o ? v : o;
    }
    return v;
}

// Code of one element (tt_metal/common/bfloat8.hpp:23-87, blockfloat_common.hpp:67-147): hidden one OR-ed in even
// for a zero exponent field, truncating shift by the exponent gap, round half up, saturate, sign dropped when the
// mantissa rounds to zero, +-0 -> 0.  The two shifts are folded into one:
//     ((m >> gap) + h) >> s  ==  (m + (h << gap)) >> (gap + s)        (h = 2^(s-1), s = 24 - W)
// and every gap above 31 - s gives 0 either way (m < 2^24), so the gap is clamped there and nothing overflows.
template <int W> __device__ __forceinline__ uint32_t to_code(uint32_t bits, uint32_t shared) {
    constexpr uint32_t s = 24 - W, h = 1u << (s - 1), top = (1u << W) - 1u;
    const uint32_t gap = min(shared - ((bits >> 23) & 0xffu), 31u - s);
    const uint32_t m24 = (bits & 0x007fffffu) | 0x00800000u;
    uint32_t m = min(((h << gap) + m24) >> (gap + s), top);
    m = (bits & 0x7fffffffu) ? m : 0u;
    return m ? (((bits >> 31) << W) | m) : 0u;
}

// Epilogue of the tiled GEMM kernels for one wavefront: a 128-row x 64-column part of C (one 64-column weight group) whose
// accumulators lie as v_mfma_f32_32x32x16 leaves them, with the column order of the weight expansion:
//   acc[rb][cb][i] = row 32 rb + 8 (i / 4) + 4 kh + i % 4, column 32 t + 16 fc + 4 q + 2 half + cb of the 64, for lane
//   (c = lane % 32, kh = lane / 32), c16 = c % 16, half = c / 16, t = c16 / 8, fc = (c16 / 4) % 2, q = c16 % 4.
// A lane therefore owns pairs of adjacent columns, 4 bytes of bf16: stored directly that is one 32- or 64-byte piece per
// row and instruction.  Instead the wavefront lays the bf16 block out in 16 KB of LDS of its own exactly as it lies in
// memory (TILE layout: per 32 rows the two tiles are 4 KB contiguous; row-major: 128 bytes per row) and copies it out
// with 16 bytes per lane.  fp32 output is stored directly (8 bytes per lane).
struct StoreTarget {
    uint8_t *c;              // output
    const uint16_t *bias;    // bf16 [n] or null
    uint32_t m, n, nt;       // rows of a batch slice, columns, n / 32
    uint64_t slice;          // batch slice
    uint32_t row0;           // first row of the part
    uint32_t nt0;            // first packed tile column of the group (the group has 1 or 2 tiles)
    float unscale;
    int c_tiled, c_f32;
    int c_bfp;               // 0, or the mantissa bits (7 | 3) of a block-float output (TILE layout)
};

template <int ACT, typename Acc, int RB>
__device__ __forceinline__ void store_wave_part(const Acc (&acc)[RB][2], const StoreTarget &o, uint8_t *lds_wave, int lane) {
    const int c = lane & 31, kh = lane >> 5;
    const int c16 = c & 15, half = c >> 4;
    const int t = c16 >> 3, fc = (c16 >> 2) & 1, q = c16 & 3;
    if (o.nt0 >= o.nt) return;
    const uint32_t tiles = min(2u, o.nt - o.nt0);
    const uint32_t col = t * 32 + fc * 16 + q * 4 + half * 2;             // of the group's 64
    const bool lane_valid = (uint32_t)t < tiles;
    float bias_v[2] = {0.f, 0.f};
    if (o.bias && lane_valid) {
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) bias_v[cb] = __uint_as_float((uint32_t)o.bias[o.nt0 * 32 + col + cb] << 16);
    }
    const uint32_t mt = (o.m + 31) / 32;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t r32 = (i >> 2) * 8 + kh * 4 + (i & 3);
            const float v0 = apply_activation<ACT>(acc[rb][0][i] * o.unscale + bias_v[0]), v1 = apply_activation<ACT>(acc[rb][1][i] * o.unscale + bias_v[1]);
            if (o.c_f32) {
                const uint32_t row = o.row0 + rb * 32 + r32;
                if (row >= o.m || !lane_valid) continue;
                uint64_t elem;
                if (o.c_tiled) elem = ((o.slice * mt + (row >> 5)) * o.nt + o.nt0 + t) * 1024 + (((row >> 4) & 1) * 2 + fc) * 256 + (row & 15) * 16 + q * 4 + half * 2;
                else elem = (o.slice * o.m + row) * o.n + o.nt0 * 32 + col;
                *reinterpret_cast<float2 *>(o.c + elem * 4) = make_float2(v0, v1);
            } else {
                const uint32_t both = f32x2_to_bf16x2_rne(v0, v1);
                // TILE layout: tile t and face column fc move a lane by 2048 and 512 bytes, i.e. onto the same banks; they are
                // XOR-ed into the two 16-byte-chunk bits that are the same for all lanes (r32 % 4), and out again below
                const uint32_t at = o.c_tiled ? rb * 4096 + t * 2048 + (((r32 >> 4) & 1) * 2 + fc) * 512 + (((r32 & 15) * 32) ^ (t * 32 + fc * 64)) + q * 8 + half * 4
                                              : (rb * 32 + r32) * 128 + col * 2;
                *reinterpret_cast<uint32_t *>(lds_wave + at) = both;
            }
        }
    }
    if (o.c_f32) return;
    if (o.c_bfp) {
        // Block-float output: the bf16 tiles staged above are packed with the host packers' arithmetic (the sums are rounded
        // to bf16 first, as for a bf16 output).  A lane takes one face row at a time — 16 bf16, 32 bytes of the stage — finds
        // the shared exponent, and writes 16 (BFLOAT8_B) or 8 (BFLOAT4_B) code bytes and the exponent byte to their places in
        // the packed tile (64 exponent bytes, then the faces' code rows: tt_metal/common/bfloat8.hpp:102-173).
        const uint32_t tile_bytes = o.c_bfp == 7 ? 1088u : 576u, row_bytes = o.c_bfp == 7 ? 16u : 8u;
#pragma unroll
        for (int it = 0; it < RB * 2; ++it) {
            const uint32_t fr = it * 64 + lane;                            // face row of the part: 32-row band, tile, face, row
            const uint32_t rb = fr >> 7, tt = (fr >> 6) & 1, f = (fr >> 4) & 3, r16 = fr & 15;
            const uint32_t row = o.row0 + rb * 32;
            if (row >= o.m || tt >= tiles) continue;
            const uint8_t *from = lds_wave + rb * 4096 + tt * 2048 + f * 512 + ((r16 * 32) ^ (tt * 32 + (f & 1) * 64));
            const u32x4 lo8 = *reinterpret_cast<const u32x4 *>(from), hi8 = *reinterpret_cast<const u32x4 *>(from + 16);
            uint32_t bits[16], shared = 0;
#pragma unroll
            for (int w2 = 0; w2 < 4; ++w2) {
                bits[2 * w2] = lo8[w2] << 16; bits[2 * w2 + 1] = lo8[w2] & 0xffff0000u;
                bits[8 + 2 * w2] = hi8[w2] << 16; bits[8 + 2 * w2 + 1] = hi8[w2] & 0xffff0000u;
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) shared = max(shared, (bits[e] >> 23) & 0xffu);
            uint8_t *tile = o.c + ((o.slice * mt + (row >> 5)) * o.nt + o.nt0 + tt) * tile_bytes;
            uint32_t words[4] = {0, 0, 0, 0};
            if (o.c_bfp == 7) {
#pragma unroll
                for (int e = 0; e < 16; ++e) words[e >> 2] |= to_code<7>(bits[e], shared) << (8 * (e & 3));
                *reinterpret_cast<u32x4 *>(tile + 64 + f * 256 + r16 * row_bytes) = u32x4{words[0], words[1], words[2], words[3]};
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) words[e >> 3] |= to_code<3>(bits[e], shared) << (4 * (e & 7));
                *reinterpret_cast<uint2 *>(tile + 64 + f * 128 + r16 * row_bytes) = make_uint2(words[0], words[1]);
            }
            tile[f * 16 + r16] = (uint8_t)shared;
        }
        return;
    }
    if (o.c_tiled) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const uint32_t row = o.row0 + rb * 32;
            if (row >= o.m) break;
            uint8_t *dst = o.c + ((o.slice * mt + (row >> 5)) * o.nt + o.nt0) * 2048;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if ((uint32_t)j < tiles * 2)
                    *reinterpret_cast<u32x4 *>(dst + j * 1024 + lane * 16) =
                        *reinterpret_cast<const u32x4 *>(lds_wave + rb * 4096 + j * 1024 + ((lane * 16) ^ ((j >> 1) * 32 + ((lane >> 5) & 1) * 64)));
        }
    } else {
        const uint32_t chunk = lane & 7;
#pragma unroll
        for (int j = 0; j < 4 * RB; ++j) {
            const uint32_t r = j * 8 + (lane >> 3), row = o.row0 + r;
            if (row < o.m && chunk < tiles * 4)
                *reinterpret_cast<u32x4 *>(o.c + ((o.slice * o.m + row) * o.n + o.nt0 * 32) * 2 + chunk * 16) =
                    *reinterpret_cast<const u32x4 *>(lds_wave + r * 128 + chunk * 16);
        }
    }
}

}  // namespace ttmi
