// Block-float codec kernels for gfx950: fused pad + tilize + pack, and unpack + untilize.
//
// Arithmetic follows tt-metal's host codecs bit for bit:
//   shared exponent   tt_metal/common/blockfloat_common.hpp:19-47   (max raw exponent field of a 16-element face row)
//   element -> code   tt_metal/common/bfloat8.hpp:23-87, blockfloat_common.hpp:67-147
//   tile layout       bfloat8.hpp:102-173 (64 exponent bytes, then faces 0..3 row by row, element 0 in the low bits)
//   code -> element   bfloat8.hpp:229-249, tt_metal/common/bfloat4.hpp:113-146
//   tilize order      tt_metal/common/test_tiles.hpp:24-65,123-158
//
// Work decomposition (HBM-bound, nothing is read twice):
//   a lane owns 16 bytes of one face row (4 fp32 or 8 bf16), LPR = 4 or 2 neighbouring lanes own the row;
//   a wavefront covers 1 KiB of contiguous source per step, a 256-thread block covers 32 rows x TPB tiles;
//   the row's shared exponent is a DPP quad-permute max over the LPR lanes;
//   packed tiles are assembled in LDS and leave (or enter) the block as one contiguous run of 16-byte accesses.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include "bfp_dequant.h"
#include "ttmi_internal.h"

namespace ttmi {

enum SrcMode { SRC_TENSOR = 0, SRC_TILE_ROWMAJOR = 1, SRC_TILE_FACES = 2 };

struct CodecShape {
    uint32_t batch, h, w;       // logical extent (SRC_TENSOR); unused for tile-chunk modes
    uint32_t ht, wt;            // tiles per column / row of the padded tensor
    uint32_t col_groups;        // ceil(wt / TPB)
    uint64_t n_tiles;           // total tiles
    uint64_t row_stride;        // elements between rows of the row-major tensor
    uint64_t batch_stride;      // elements between [h, w] slices
};

template <int W> struct Fmt;
template <> struct Fmt<7> { static constexpr int tile_bytes = 1088, row_bytes = 16, face_bytes = 256; };
template <> struct Fmt<3> { static constexpr int tile_bytes = 576, row_bytes = 8, face_bytes = 128; };

// row_max (shared exponent of a face row over its lanes) and to_code (one element's code) live in bfp_dequant.h
template <int W> __device__ __forceinline__ uint32_t from_code(uint32_t code, uint32_t shared) {
    const uint32_t man = code & ((1u << W) - 1u);
    const uint32_t sign = ((code >> W) & 1u) << 31;
    const int sc = __clz((int)man) - (32 - W);
    const uint32_t frac = (man << (sc + 1)) & ((1u << W) - 1u);
    const uint32_t ex = (uint32_t)((int)shared - sc);
    const uint32_t bits = sign | (ex << 23) | (frac << (23 - W));
    return man ? bits : sign;
}

// Which (tile-in-block, face, row-in-face, lane-in-row) a lane handles at step `it`, and where its 16 source
// bytes live.  ELEM = bytes per source element.  A block of 256 threads covers 32 rows x TPB tiles; TPB is 8 (fp32) or
// 16 (bf16) halved SHRINK times: small tensors are cut into more, narrower blocks so that the grid still fills the chip.
template <int ELEM, int SHRINK = 0> struct Item {
    static constexpr int LPR = ELEM;               // lanes per face row: 4 (fp32) or 2 (bf16)
    static constexpr int EPL = 16 / ELEM;          // elements per lane: 4 or 8
    static constexpr int TPB = (32 / LPR) >> SHRINK;   // tiles per block
    static constexpr int ITS = 8 >> SHRINK;        // steps per wavefront, one KiB of source each
    static constexpr int LANES_PER_ROW = TPB * 2 * LPR;            // 64, 32 or 16 lanes walk along one tensor row
    static constexpr int ROWS_PER_STEP = 64 / LANES_PER_ROW;
    int t, face, i, q;
    __device__ __forceinline__ Item(int mode, int wave, int it, int lane) {
        const int step = wave * ITS + it;
        q = lane % LPR;
        if (mode == SRC_TENSOR) {                  // the wave walks along ROWS_PER_STEP tensor rows
            const int r = step * ROWS_PER_STEP + lane / LANES_PER_ROW;
            const int within = lane % LANES_PER_ROW;
            t = within / (2 * LPR);
            face = (r >> 4) * 2 + ((within / LPR) & 1);
            i = r & 15;
        } else {                                   // the wave walks through the block's contiguous chunks
            if (ELEM == 4) {                       // tile = 4 KiB = 4 steps
                t = step >> 2;
                const int part = step & 3;
                if (mode == SRC_TILE_FACES) { face = part; i = lane >> 2; }
                else { const int r = part * 8 + (lane >> 3); face = (r >> 4) * 2 + ((lane >> 2) & 1); i = r & 15; }
            } else {                               // tile = 2 KiB = 2 steps
                t = step >> 1;
                const int part = step & 1;
                if (mode == SRC_TILE_FACES) { face = part * 2 + (lane >> 5); i = (lane >> 1) & 15; }
                else { const int r = part * 16 + (lane >> 2); face = (r >> 4) * 2 + ((lane >> 1) & 1); i = r & 15; }
            }
        }
    }
};

template <int ELEM> __device__ __forceinline__ void expand(const uint4 raw, uint32_t (&bits)[16 / ELEM]) {
    if (ELEM == 4) {
        bits[0] = raw.x; bits[1] = raw.y; bits[2] = raw.z; bits[3] = raw.w;
    } else {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) { bits[2 * k] = w[k] << 16; bits[2 * k + 1] = w[k] & 0xffff0000u; }
    }
}

// Codes of a lane's 16 source bytes in an ordinary face row (shared exponent 32 <= E < 255, every element a normal float or
// zero; or a row of nothing but zeros), lowest element in the lowest bits of lo (bfp8 from bf16: elements 4..7 in hi).
// The packers' recipe (shift the 24-bit mantissa down by the exponent gap, add half, shift again) is
//     floor(v + 1/2),  v = |x| * 2^(126+W-E)  (an exact product)   ==   trunc(fma(|x|, 2^(126+W-E), 1/2 - 2^-25))
// for every 24-bit mantissa and every exponent gap: the fma rounds the exact sum once, to nearest even, which never crosses
// an integer (with 1/2 itself the single case v = 1/2 - 2^-25 would round up to 1).  v + 1/2 < 2^W + 1/2, so a code exceeds
// 2^W - 1 only by being 2^W.  Saturation, the sign (bit 7 of the element's top byte) and "no sign on a zero mantissa" are
// applied to four codes, one per byte, at a time.
template <int W, int ELEM> __device__ __forceinline__ void ordinary_codes(const uint4 raw, uint32_t shared, uint32_t &lo, uint32_t &hi) {
    constexpr int EPL = 16 / ELEM;
    constexpr uint32_t ONES = 0x01010101u, TOP = ONES << W, LOW = TOP - ONES;       // per byte: 2^W, 2^W - 1
    uint32_t bits[EPL];
    expand<ELEM>(raw, bits);
    const float scale = shared < 32u ? 0.f : __uint_as_float((253u + (uint32_t)W - shared) << 23);
    uint32_t c4[EPL / 4];
#pragma unroll
    for (int g = 0; g < EPL / 4; ++g) {
        uint32_t m4 = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            m4 |= (uint32_t)__builtin_fmaf(fabsf(__uint_as_float(bits[4 * g + e])), scale, 0.5f - 0x1p-25f) << (8 * e);
        uint32_t sign4;
        if (ELEM == 4) sign4 = __builtin_amdgcn_perm(raw.y, raw.x, 0x0c0c0703u) | __builtin_amdgcn_perm(raw.w, raw.z, 0x07030c0cu);
        else sign4 = g == 0 ? __builtin_amdgcn_perm(raw.y, raw.x, 0x07050301u) : __builtin_amdgcn_perm(raw.w, raw.z, 0x07050301u);
        m4 -= (m4 & TOP) >> W;                                   // 2^W -> 2^W - 1
        const uint32_t nonzero = m4 + LOW;                       // bit W of a byte set iff its code is not zero
        c4[g] = (((W == 7 ? sign4 : sign4 >> 4) & nonzero) & TOP) | m4;
        if (W == 3) {                                            // the low nibbles of the four bytes -> 16 bits
            const uint32_t pairs = c4[g] | (c4[g] >> 4);         // bytes 0 and 2 hold a pair each
            c4[g] = __builtin_amdgcn_perm(0u, pairs, 0x0c0c0200u);
        }
    }
    if (W == 7) { lo = c4[0]; hi = c4[EPL / 4 - 1]; }
    else { lo = EPL == 4 ? c4[0] : (c4[0] | (c4[EPL / 4 - 1] << 16)); hi = 0u; }
}

// ---------------------------------------------------------------------------------------------------------
// pack: MODE selects how the source is addressed; ALIGNED means every lane may use one 16-byte load.
// ---------------------------------------------------------------------------------------------------------
template <int W, int ELEM, int MODE, bool ALIGNED, int SHRINK = 0>
__global__ __launch_bounds__(256) void pack_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                   const CodecShape s) {
    using F = Fmt<W>;
    using I = Item<ELEM, SHRINK>;
    constexpr int TPB = I::TPB, EPL = I::EPL, LPR = I::LPR, ITS = I::ITS;
    __shared__ __attribute__((aligned(16))) uint8_t stage[TPB * F::tile_bytes];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint64_t tile0;          // first tile of this block in the output
    uint32_t n_valid;        // tiles of this block that exist
    uint32_t row0 = 0, col0 = 0;
    const uint8_t *slice = src;
    if (MODE == SRC_TENSOR) {
        const uint32_t cg = blockIdx.x % s.col_groups;
        const uint64_t rest = blockIdx.x / s.col_groups;
        const uint32_t tr = (uint32_t)(rest % s.ht);
        const uint64_t b = rest / s.ht;
        tile0 = (b * s.ht + tr) * s.wt + (uint64_t)cg * TPB;
        n_valid = min((uint32_t)TPB, s.wt - cg * TPB);
        row0 = tr * 32; col0 = cg * TPB * 32;
        slice = src + b * s.batch_stride * ELEM;
    } else {
        tile0 = (uint64_t)blockIdx.x * TPB;
        n_valid = (uint32_t)min((uint64_t)TPB, s.n_tiles - tile0);
    }

    uint4 raw[ITS];
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        const I at(MODE, wave, it, lane);
        raw[it] = make_uint4(0, 0, 0, 0);
        if (at.t >= (int)n_valid) continue;
        if (MODE == SRC_TENSOR) {
            const uint32_t r = row0 + (at.face >> 1) * 16 + at.i;
            const uint32_t c = col0 + at.t * 32 + (at.face & 1) * 16 + at.q * EPL;
            if (r >= s.h || c >= s.w) continue;
            const uint8_t *p = slice + ((uint64_t)r * s.row_stride + c) * ELEM;
            if (ALIGNED) {
                raw[it] = *reinterpret_cast<const uint4 *>(p);
            } else {
                uint32_t tmp[4] = {0, 0, 0, 0};
                for (int e = 0; e < EPL; ++e)
                    if (c + e < s.w) {
                        if (ELEM == 4) tmp[e] = reinterpret_cast<const uint32_t *>(p)[e];
                        else tmp[e >> 1] |= (uint32_t) reinterpret_cast<const uint16_t *>(p)[e] << (16 * (e & 1));
                    }
                raw[it] = make_uint4(tmp[0], tmp[1], tmp[2], tmp[3]);
            }
        } else {
            const uint64_t chunk = (tile0 + at.t) * 1024 * ELEM;
            const int within = MODE == SRC_TILE_FACES ? (at.face * 256 + at.i * 16 + at.q * EPL)
                                                      : (((at.face >> 1) * 16 + at.i) * 32 + (at.face & 1) * 16 + at.q * EPL);
            raw[it] = *reinterpret_cast<const uint4 *>(src + chunk + (uint64_t)within * ELEM);
        }
    }

    // Shared exponents of the wavefront's eight face-row pieces first, and with them one question for the whole wavefront:
    // is every row ordinary?  A row is ordinary if its exponent is 32 <= E < 255 (all elements normal floats or zero; no
    // Inf or NaN), or if it holds nothing but zeros: ordinary_codes then gives the packers' codes by float arithmetic.
    // Everything else (non-zero values below 2^-95, where the reference ORs a hidden one into subnormals and from_torch's
    // double pass zeroes single-bit codes; Inf; NaN) sends the wavefront through the integer recipe.  One ballot per
    // wavefront: per-item ballots and the branches behind them cost 2 to 4 us of 18 for a 4096 x 4096 tensor.
    uint32_t shared_of[ITS];
    bool odd = false;
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        uint32_t bits[EPL];
        expand<ELEM>(raw[it], bits);
        uint32_t top = 0, nonzero = 0;
#pragma unroll
        for (int e = 0; e < EPL; ++e) { const uint32_t f = bits[e] & 0x7f800000u; top = f > top ? f : top; nonzero |= bits[e]; }
        shared_of[it] = row_max<LPR>(top) >> 23;
        odd |= (shared_of[it] < 32u && (nonzero & 0x7fffffffu) != 0) || shared_of[it] == 255u;
    }
    const bool ordinary = __ballot(odd) == 0;

    auto put = [&](const I &at, uint32_t shared, uint32_t lo, uint32_t hi) __attribute__((always_inline)) {
        if (at.t < (int)n_valid) {
            uint8_t *tile = stage + at.t * F::tile_bytes;
            if (at.q == 0) tile[at.face * 16 + at.i] = (uint8_t)shared;
            uint8_t *row = tile + 64 + at.face * F::face_bytes + at.i * F::row_bytes;
            constexpr int lane_bytes = EPL * (W + 1) / 8;          // 4, 8 (bfp8) or 2, 4 (bfp4)
            if (lane_bytes == 2) reinterpret_cast<uint16_t *>(row)[at.q] = (uint16_t)lo;
            else if (lane_bytes == 4) reinterpret_cast<uint32_t *>(row)[at.q] = lo;
            else reinterpret_cast<uint2 *>(row)[at.q] = make_uint2(lo, hi);
        }
    };
    if (ordinary) {
#pragma unroll
        for (int it = 0; it < ITS; ++it) {
            const I at(MODE, wave, it, lane);
            uint32_t lo, hi;
            ordinary_codes<W, ELEM>(raw[it], shared_of[it], lo, hi);
            put(at, shared_of[it], lo, hi);
        }
    } else {
#pragma unroll
        for (int it = 0; it < ITS; ++it) {
            const I at(MODE, wave, it, lane);
            uint32_t bits[EPL];
            expand<ELEM>(raw[it], bits);
            const uint32_t shared = shared_of[it];
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                uint32_t code = to_code<W>(bits[e], shared);
                // from_torch runs pack -> unpack -> tilize -> pack (tt_eager/tensor/tensor_impl.cpp:179-197).  A code
                // whose mantissa is the single bit 2^(W-1-E) unpacks to exponent field 0 with a zero fraction, i.e.
                // to +-0, and the second pack turns that into code 0; every other code survives the round trip.
                // Only rows with E < W (magnitudes below 2^-120) can be hit.
                if (MODE == SRC_TENSOR && shared < (uint32_t)W && (code & ((1u << W) - 1u)) == (1u << ((W - 1 - shared) & 31u))) code = 0;
                const int sh = (W + 1) * e;
                if (sh < 32) lo |= code << sh; else hi |= code << (sh - 32);
            }
            put(at, shared, lo, hi);
        }
    }
    __syncthreads();
    const uint32_t n16 = n_valid * (F::tile_bytes / 16);
    uint4 *out = reinterpret_cast<uint4 *>(dst + tile0 * F::tile_bytes);
    const uint4 *in = reinterpret_cast<const uint4 *>(stage);
    for (uint32_t k = threadIdx.x; k < n16; k += 256) out[k] = in[k];
}

// ---------------------------------------------------------------------------------------------------------
// pack of a row-major tensor whose blocks are all whole (h a multiple of 32, w a multiple of the block width, every lane
// may use one 16-byte load): the same walk as pack_kernel<.., SRC_TENSOR, true, 0> in straight-line code.  Wavefront `wave`
// reads rows 8 wave .. 8 wave + 7 of the block, one row (1 KiB) per load; lane = (tile, face column, quarter or half of the
// face row), the same for all eight rows, so everything but the row is fixed per lane, the LDS addresses of the eight
// items differ by constants and the eight exponent bytes of a lane are one 8-byte store.  An item is processed as soon as
// its load has landed; a wavefront with a row that is not ordinary redoes its eight items with the integer recipe.
// ---------------------------------------------------------------------------------------------------------
template <int W, int ELEM>
__global__ __launch_bounds__(256) void pack_whole_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                         const CodecShape s) {
    using F = Fmt<W>;
    using I = Item<ELEM, 0>;
    constexpr int TPB = I::TPB, EPL = I::EPL, LPR = I::LPR, ITS = 8;
    constexpr int lane_bytes = EPL * (W + 1) / 8;               // 4, 8 (bfp8) or 2, 4 (bfp4)
    __shared__ __attribute__((aligned(16))) uint8_t stage[TPB * F::tile_bytes];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t cg = blockIdx.x % s.col_groups;
    const uint64_t rest = blockIdx.x / s.col_groups;
    const uint32_t tr = (uint32_t)(rest % s.ht);
    const uint64_t b = rest / s.ht;
    const uint64_t tile0 = (b * s.ht + tr) * s.wt + (uint64_t)cg * TPB;
    const uint8_t *p = src + (b * s.batch_stride + (uint64_t)(tr * 32 + wave * 8) * s.row_stride + (uint64_t)cg * TPB * 32) * ELEM + lane * 16;

    uint4 raw[ITS];
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        // read once: the non-temporal policy keeps the 64 MiB of a large source from displacing what the caches hold
        // (measured on fp32 4096 x 4096 -> BFLOAT4_B: 13.6 against 14.1 us)
        typedef uint32_t v4 __attribute__((ext_vector_type(4)));
        const v4 v = __builtin_nontemporal_load(reinterpret_cast<const v4 *>(p + (uint64_t)it * s.row_stride * ELEM));
        raw[it] = make_uint4(v.x, v.y, v.z, v.w);
    }

    const int t = lane / (2 * LPR), fc = (lane / LPR) & 1, q = lane % LPR;
    const int face = (wave >> 1) * 2 + fc, i0 = (wave & 1) * 8;
    uint8_t *tile = stage + t * F::tile_bytes;
    uint8_t *row0 = tile + 64 + face * F::face_bytes + i0 * F::row_bytes + q * lane_bytes;

    auto put = [&](int it, uint32_t lo, uint32_t hi) __attribute__((always_inline)) {
        uint8_t *row = row0 + it * F::row_bytes;
        if (lane_bytes == 2) *reinterpret_cast<uint16_t *>(row) = (uint16_t)lo;
        else if (lane_bytes == 4) *reinterpret_cast<uint32_t *>(row) = lo;
        else *reinterpret_cast<uint2 *>(row) = make_uint2(lo, hi);
    };
    uint32_t exps[2] = {0u, 0u};
    bool odd = false;
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        uint32_t bits[EPL];
        expand<ELEM>(raw[it], bits);
        uint32_t top = 0;                                        // largest |x| of the lane, as bits shifted up by one
#pragma unroll
        for (int e = 0; e < EPL; ++e) { const uint32_t a = bits[e] << 1; top = a > top ? a : top; }
        top = row_max<LPR>(top);
        const uint32_t shared = top >> 24;
        odd |= (shared < 32u && top != 0u) || shared == 255u;
        exps[it >> 2] |= shared << (8 * (it & 3));
        uint32_t lo, hi;
        ordinary_codes<W, ELEM>(raw[it], shared, lo, hi);
        put(it, lo, hi);
    }
    if (q == 0) *reinterpret_cast<uint2 *>(tile + face * 16 + i0) = make_uint2(exps[0], exps[1]);

    if (__ballot(odd) != 0) {                                    // the integer recipe, as in pack_kernel
#pragma unroll
        for (int it = 0; it < ITS; ++it) {
            uint32_t bits[EPL];
            expand<ELEM>(raw[it], bits);
            const uint32_t shared = (exps[it >> 2] >> (8 * (it & 3))) & 0xffu;
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                uint32_t code = to_code<W>(bits[e], shared);
                if (shared < (uint32_t)W && (code & ((1u << W) - 1u)) == (1u << ((W - 1 - shared) & 31u))) code = 0;
                const int sh = (W + 1) * e;
                if (sh < 32) lo |= code << sh; else hi |= code << (sh - 32);
            }
            put(it, lo, hi);
        }
    }
    __syncthreads();
    constexpr uint32_t n16 = TPB * (F::tile_bytes / 16);
    uint4 *out = reinterpret_cast<uint4 *>(dst + tile0 * F::tile_bytes);
    const uint4 *in = reinterpret_cast<const uint4 *>(stage);
#pragma unroll
    for (uint32_t k = threadIdx.x; k < n16; k += 256) out[k] = in[k];
}

// ---------------------------------------------------------------------------------------------------------
// unpack: the inverse walk.  ELEM is the destination element size (4 = fp32, 2 = bf16).
// ---------------------------------------------------------------------------------------------------------
template <int W, int ELEM, int MODE, bool ALIGNED, int SHRINK = 0>
__global__ __launch_bounds__(256) void unpack_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                     const CodecShape s) {
    using F = Fmt<W>;
    using I = Item<ELEM, SHRINK>;
    constexpr int TPB = I::TPB, EPL = I::EPL, ITS = I::ITS;
    __shared__ __attribute__((aligned(16))) uint8_t stage[TPB * F::tile_bytes];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint64_t tile0;
    uint32_t n_valid;
    uint32_t row0 = 0, col0 = 0;
    uint8_t *slice = dst;
    if (MODE == SRC_TENSOR) {
        const uint32_t cg = blockIdx.x % s.col_groups;
        const uint64_t rest = blockIdx.x / s.col_groups;
        const uint32_t tr = (uint32_t)(rest % s.ht);
        const uint64_t b = rest / s.ht;
        tile0 = (b * s.ht + tr) * s.wt + (uint64_t)cg * TPB;
        n_valid = min((uint32_t)TPB, s.wt - cg * TPB);
        row0 = tr * 32; col0 = cg * TPB * 32;
        slice = dst + b * s.batch_stride * ELEM;
    } else {
        tile0 = (uint64_t)blockIdx.x * TPB;
        n_valid = (uint32_t)min((uint64_t)TPB, s.n_tiles - tile0);
    }
    {
        const uint32_t n16 = n_valid * (F::tile_bytes / 16);
        const uint4 *in = reinterpret_cast<const uint4 *>(src + tile0 * F::tile_bytes);
        uint4 *out = reinterpret_cast<uint4 *>(stage);
        for (uint32_t k = threadIdx.x; k < n16; k += 256) out[k] = in[k];
    }
    __syncthreads();

#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        const I at(MODE, wave, it, lane);
        if (at.t >= (int)n_valid) continue;
        const uint8_t *tile = stage + at.t * F::tile_bytes;
        const uint32_t shared = tile[at.face * 16 + at.i];
        const uint8_t *row = tile + 64 + at.face * F::face_bytes + at.i * F::row_bytes;
        constexpr int lane_bytes = EPL * (W + 1) / 8;
        uint32_t lo, hi = 0;
        if (lane_bytes == 2) lo = reinterpret_cast<const uint16_t *>(row)[at.q];
        else if (lane_bytes == 4) lo = reinterpret_cast<const uint32_t *>(row)[at.q];
        else { const uint2 v = reinterpret_cast<const uint2 *>(row)[at.q]; lo = v.x; hi = v.y; }
        uint32_t bits[EPL];
        // Where the result is an ordinary float, i.e. W <= E < 248, the unpacker's normalisation (count leading zeros, shift,
        // assemble) is the float arithmetic mantissa * 2^(E - 126 - W), exact because the mantissa has at most 7 bits:
        // convert, multiply by a power of two, put the sign on.  Rows outside that range (non-zero values below 2^-120, where
        // the reference's exponent subtraction wraps, or near overflow) take the integer route, a wavefront at a time.
        // (a row of zeros, E = 0 with no mantissa bit set, is ordinary: it comes out as signed zeros either way)
        constexpr uint32_t all_mantissas = W == 7 ? 0x7f7f7f7fu : 0x77777777u;
        const bool tiny = shared < (uint32_t)W;
        const bool odd_rows = __ballot((tiny && ((lo | hi) & all_mantissas) != 0) || shared >= 248u) != 0;
        const float two_to = tiny ? 0.f : __uint_as_float((shared - (uint32_t)W + 1u) << 23);
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            const int sh = (W + 1) * e;
            const uint32_t field = sh < 32 ? (lo >> sh) : (hi >> (sh - 32));            // the code in its low W + 1 bits
            if (!odd_rows) {
                const float magnitude = (float)(field & ((1u << W) - 1u)) * two_to;
                bits[e] = __float_as_uint(magnitude) | ((field << (31 - W)) & 0x80000000u);
                // to_torch runs unpack -> untilize -> pack -> unpack: a sign-only value (code 0x80 / 0x8, which no
                // packer writes) is packed to code 0 on the way and comes out as +0.0f; -0 + 0 is +0, all else stays
                if (MODE == SRC_TENSOR) bits[e] = __float_as_uint(__uint_as_float(bits[e]) + 0.0f);
            } else {
                bits[e] = from_code<W>(field & ((2u << W) - 1u), shared);
                if (MODE == SRC_TENSOR && (bits[e] & 0x7fffffffu) == 0) bits[e] = 0;
            }
        }
        uint4 v;
        if (ELEM == 4) v = make_uint4(bits[0], bits[1], bits[2], bits[3]);
        else v = make_uint4((bits[0] >> 16) | (bits[1 % EPL] & 0xffff0000u), (bits[2 % EPL] >> 16) | (bits[3 % EPL] & 0xffff0000u),
                            (bits[4 % EPL] >> 16) | (bits[5 % EPL] & 0xffff0000u), (bits[6 % EPL] >> 16) | (bits[7 % EPL] & 0xffff0000u));
        if (MODE == SRC_TENSOR) {
            const uint32_t r = row0 + (at.face >> 1) * 16 + at.i;
            const uint32_t c = col0 + at.t * 32 + (at.face & 1) * 16 + at.q * EPL;
            if (r >= s.h || c >= s.w) continue;
            uint8_t *p = slice + ((uint64_t)r * s.row_stride + c) * ELEM;
            if (ALIGNED) {
                *reinterpret_cast<uint4 *>(p) = v;
            } else {
                for (int e = 0; e < EPL; ++e)
                    if (c + e < s.w) {
                        if (ELEM == 4) reinterpret_cast<uint32_t *>(p)[e] = bits[e];
                        else reinterpret_cast<uint16_t *>(p)[e] = (uint16_t)(bits[e] >> 16);
                    }
            }
        } else {
            const uint64_t chunk = (tile0 + at.t) * 1024 * ELEM;
            const int within = MODE == SRC_TILE_FACES ? (at.face * 256 + at.i * 16 + at.q * EPL)
                                                      : (((at.face >> 1) * 16 + at.i) * 32 + (at.face & 1) * 16 + at.q * EPL);
            *reinterpret_cast<uint4 *>(dst + chunk + (uint64_t)within * ELEM) = v;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// unpack into a row-major tensor whose blocks are all whole: the walk of pack_whole_kernel backwards, in straight-line code.
// A lane's eight face rows (rows 8 wave .. 8 wave + 7 of the block, same tile, face column and piece of the row) have their
// exponents in eight consecutive bytes and their codes a constant number of bytes apart.  The decision "is every row of the
// wavefront ordinary" (see unpack_kernel) is taken once, from the eight exponents and code words; ordinary rows are
//     fma(mantissa, +-2^(E - 126 - W), +0.0)
// (the mantissa converted from its byte or bit field, the sign moved onto the power of two; the +0.0 of the to_torch
// sequence is the fma's addend: a sign-only code comes out as -0 + 0 = +0), other wavefronts take the integer route.
// ---------------------------------------------------------------------------------------------------------
template <int W, int ELEM>
__global__ __launch_bounds__(256) void unpack_whole_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                           const CodecShape s) {
    using F = Fmt<W>;
    using I = Item<ELEM, 0>;
    constexpr int TPB = I::TPB, EPL = I::EPL, LPR = I::LPR, ITS = 8;
    constexpr int lane_bytes = EPL * (W + 1) / 8;               // 4, 8 (bfp8) or 2, 4 (bfp4)
    __shared__ __attribute__((aligned(16))) uint8_t stage[TPB * F::tile_bytes];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t cg = blockIdx.x % s.col_groups;
    const uint64_t rest = blockIdx.x / s.col_groups;
    const uint32_t tr = (uint32_t)(rest % s.ht);
    const uint64_t b = rest / s.ht;
    const uint64_t tile0 = (b * s.ht + tr) * s.wt + (uint64_t)cg * TPB;
    {
        constexpr uint32_t n16 = TPB * (F::tile_bytes / 16);
        const uint4 *in = reinterpret_cast<const uint4 *>(src + tile0 * F::tile_bytes);
        uint4 *out = reinterpret_cast<uint4 *>(stage);
#pragma unroll
        for (uint32_t k = threadIdx.x; k < n16; k += 256) {      // read once: non-temporal (13.0 against 13.4 us for BFLOAT4_B -> fp32 4096 x 4096)
            typedef uint32_t v4 __attribute__((ext_vector_type(4)));
            const v4 v = __builtin_nontemporal_load(reinterpret_cast<const v4 *>(in + k));
            out[k] = make_uint4(v.x, v.y, v.z, v.w);
        }
    }
    __syncthreads();

    const int t = lane / (2 * LPR), fc = (lane / LPR) & 1, q = lane % LPR;
    const int face = (wave >> 1) * 2 + fc, i0 = (wave & 1) * 8;
    const uint8_t *tile = stage + t * F::tile_bytes;
    const uint8_t *row0 = tile + 64 + face * F::face_bytes + i0 * F::row_bytes + q * lane_bytes;
    const uint2 exps = *reinterpret_cast<const uint2 *>(tile + face * 16 + i0);
    uint32_t lo[ITS], hi[ITS];
    bool odd = false;
    constexpr uint32_t all_mantissas = W == 7 ? 0x7f7f7f7fu : 0x77777777u;
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        const uint8_t *row = row0 + it * F::row_bytes;
        hi[it] = 0;
        if (lane_bytes == 2) lo[it] = *reinterpret_cast<const uint16_t *>(row);
        else if (lane_bytes == 4) lo[it] = *reinterpret_cast<const uint32_t *>(row);
        else { const uint2 v = *reinterpret_cast<const uint2 *>(row); lo[it] = v.x; hi[it] = v.y; }
        const uint32_t shared = ((it < 4 ? exps.x : exps.y) >> (8 * (it & 3))) & 0xffu;
        odd |= (shared < (uint32_t)W && ((lo[it] | hi[it]) & all_mantissas) != 0) || shared >= 248u;
    }
    const bool odd_rows = __ballot(odd) != 0;
    uint8_t *p = dst + (b * s.batch_stride + (uint64_t)(tr * 32 + wave * 8) * s.row_stride + (uint64_t)cg * TPB * 32) * ELEM + lane * 16;
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        const uint32_t shared = ((it < 4 ? exps.x : exps.y) >> (8 * (it & 3))) & 0xffu;
        uint32_t bits[EPL];
        if (!odd_rows) {
            const uint32_t two_to = shared < (uint32_t)W ? 0u : (shared - (uint32_t)W + 1u) << 23;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int sh = (W + 1) * e;
                const uint32_t word = sh < 32 ? lo[it] : hi[it];
                const int at = sh & 31;                                               // the code's lowest bit in its word
                const float mantissa = (float)((word >> at) & ((1u << W) - 1u));
                const uint32_t sign = at + W == 31 ? word : word << (31 - W - at);    // the sign bit moved to bit 31
                bits[e] = __float_as_uint(__builtin_fmaf(mantissa, __uint_as_float((sign & 0x80000000u) | two_to), 0.0f));
            }
        } else {
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int sh = (W + 1) * e;
                const uint32_t field = sh < 32 ? (lo[it] >> sh) : (hi[it] >> (sh - 32));
                bits[e] = from_code<W>(field & ((2u << W) - 1u), shared);
                if ((bits[e] & 0x7fffffffu) == 0) bits[e] = 0;
            }
        }
        uint4 v;
        if (ELEM == 4) v = make_uint4(bits[0], bits[1], bits[2], bits[3]);
        else v = make_uint4((bits[0] >> 16) | (bits[1 % EPL] & 0xffff0000u), (bits[2 % EPL] >> 16) | (bits[3 % EPL] & 0xffff0000u),
                            (bits[4 % EPL] >> 16) | (bits[5 % EPL] & 0xffff0000u), (bits[6 % EPL] >> 16) | (bits[7 % EPL] & 0xffff0000u));
        *reinterpret_cast<uint4 *>(p + (uint64_t)it * s.row_stride * ELEM) = v;      // (non-temporal stores here: 14.6 against 13.0 us)
    }
}

// ---------------------------------------------------------------------------------------------------------
// tilize / untilize: pure permutation with zero padding (TO_TILES) or cropping.
// ---------------------------------------------------------------------------------------------------------
template <int ELEM, bool TO_TILES, bool ALIGNED>
__global__ __launch_bounds__(256) void relayout_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                       const CodecShape s) {
    using I = Item<ELEM>;
    constexpr int TPB = I::TPB, EPL = I::EPL;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t cg = blockIdx.x % s.col_groups;
    const uint64_t rest = blockIdx.x / s.col_groups;
    const uint32_t tr = (uint32_t)(rest % s.ht);
    const uint64_t b = rest / s.ht;
    const uint64_t tile0 = (b * s.ht + tr) * s.wt + (uint64_t)cg * TPB;
    const uint32_t n_valid = min((uint32_t)TPB, s.wt - cg * TPB);
    const uint8_t *rm_c = (TO_TILES ? src : dst) + b * s.batch_stride * ELEM;
    uint8_t *tiles = const_cast<uint8_t *>(TO_TILES ? dst : src);

    uint4 v[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const I at(SRC_TENSOR, wave, it, lane);
        v[it] = make_uint4(0, 0, 0, 0);
        if (at.t >= (int)n_valid) continue;
        const uint32_t r = tr * 32 + (at.face >> 1) * 16 + at.i;
        const uint32_t c = (cg * TPB + at.t) * 32 + (at.face & 1) * 16 + at.q * EPL;
        uint8_t *tp = tiles + ((tile0 + at.t) * 1024 + at.face * 256 + at.i * 16 + at.q * EPL) * ELEM;
        uint8_t *rp = const_cast<uint8_t *>(rm_c) + ((uint64_t)r * s.row_stride + c) * ELEM;
        if (TO_TILES) {
            if (r < s.h && c < s.w) {
                if (ALIGNED) v[it] = *reinterpret_cast<const uint4 *>(rp);
                else {
                    uint8_t tmp[16] = {0};
                    for (int e = 0; e < EPL * ELEM; ++e) if (c + e / ELEM < s.w) tmp[e] = rp[e];
                    v[it] = *reinterpret_cast<uint4 *>(tmp);
                }
            }
            *reinterpret_cast<uint4 *>(tp) = v[it];
        } else {
            if (r >= s.h || c >= s.w) continue;
            v[it] = *reinterpret_cast<const uint4 *>(tp);
            if (ALIGNED) *reinterpret_cast<uint4 *>(rp) = v[it];
            else {
                const uint8_t *tmp = reinterpret_cast<const uint8_t *>(&v[it]);
                for (int e = 0; e < EPL * ELEM; ++e) if (c + e / ELEM < s.w) rp[e] = tmp[e];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// pad / unpad of 4-D row-major data: dst[i] = src[i - offset] where that lies inside src, a fill value elsewhere
// (tt_eager/tensor/tensor_impl.hpp:508-578 pad, :609-660 unpad: offset = input_tensor_start, or minus output_tensor_start).
// ---------------------------------------------------------------------------------------------------------
struct WindowDev { uint32_t src[4], dst[4]; int32_t off[4]; };

// flat source index of flat destination index `o`, or -1 outside the source
__device__ __forceinline__ int64_t window_source(const WindowDev &w, uint64_t o) {
    int64_t at = 0;
    uint64_t stride = 1;
    bool inside = true;
#pragma unroll
    for (int d = 3; d >= 0; --d) {
        const int64_t c = (int64_t)(o % w.dst[d]) - w.off[d];
        o /= w.dst[d];
        inside = inside && c >= 0 && c < (int64_t)w.src[d];
        at += c * (int64_t)stride;
        stride *= w.src[d];
    }
    return inside ? at : -1;
}

// an element is `inner` consecutive values of T (1 for scalars; the 32-bit words of a tile when whole tiles are moved)
template <typename T>
__global__ __launch_bounds__(256) void window_copy_kernel(const T *__restrict__ src, T *__restrict__ dst, const WindowDev w, T fill, uint32_t inner,
                                                          uint64_t total) {
    for (uint64_t o = (uint64_t)blockIdx.x * 256 + threadIdx.x; o < total; o += (uint64_t)gridDim.x * 256) {
        const uint64_t elem = inner == 1 ? o : o / inner;
        const int64_t i = window_source(w, elem);
        dst[o] = i >= 0 ? src[(uint64_t)i * inner + (o - elem * inner)] : fill;
    }
}

// The same for block-float tensors declared ROW_MAJOR (consecutive 1024-element chunks of the row-major data, packed in
// sequence: tt_eager/tt_lib/csrc/tt_lib_bindings_tensor_pytensor.cpp:145-151), as tensor_impl.cpp:200-283 does it — unpack
// to fp32, pad / unpad, pack again — in one pass: a thread owns one run of 16 output elements (one shared exponent),
// decodes the source codes under it and encodes the run.
template <int W>
__global__ __launch_bounds__(256) void window_copy_bfp_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, const WindowDev w,
                                                              uint32_t fill_bits, uint64_t runs) {
    using F = Fmt<W>;
    for (uint64_t r = (uint64_t)blockIdx.x * 256 + threadIdx.x; r < runs; r += (uint64_t)gridDim.x * 256) {
        uint32_t bits[16], shared = 0;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int64_t i = window_source(w, r * 16 + e);
            uint32_t v = fill_bits;
            if (i >= 0) {
                const uint8_t *tile = src + (uint64_t)(i >> 10) * F::tile_bytes;
                const uint32_t at = (uint32_t)i & 1023u;
                const uint32_t code = W == 7 ? tile[64 + at] : (tile[64 + (at >> 1)] >> (4 * (at & 1))) & 0xfu;
                v = from_code<W>(code, tile[at >> 4]);
            }
            bits[e] = v;
            shared = max(shared, (v >> 23) & 0xffu);
        }
        uint8_t *tile = dst + (r >> 6) * F::tile_bytes;
        const uint32_t k = (uint32_t)r & 63u;
        tile[k] = (uint8_t)shared;
        uint32_t out[4] = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const uint32_t code = to_code<W>(bits[e], shared);
            if (W == 7) out[e >> 2] |= code << (8 * (e & 3));
            else out[e >> 3] |= code << (4 * (e & 7));
        }
        if (W == 7) *reinterpret_cast<uint4 *>(tile + 64 + k * 16) = make_uint4(out[0], out[1], out[2], out[3]);
        else *reinterpret_cast<uint2 *>(tile + 64 + k * 8) = make_uint2(out[0], out[1]);
    }
}

// ---------------------------------------------------------------------------------------------------------
// host launchers
// ---------------------------------------------------------------------------------------------------------
int codec_copy_window(int dtype, const void *src, const uint32_t src_shape[4], void *dst, const uint32_t dst_shape[4],
                      const int32_t offset[4], float fill, hipStream_t st) {
    WindowDev w{};
    uint64_t total = 1, src_total = 1;
    for (int d = 0; d < 4; ++d) {
        w.src[d] = src_shape[d]; w.dst[d] = dst_shape[d]; w.off[d] = offset[d];
        total *= dst_shape[d]; src_total *= src_shape[d];
    }
    if (total == 0) return TTMI_OK;
    if (total >> 40 || src_total >> 40) return fail(TTMI_ERR_INVALID_ARGUMENT, "pad / unpad: tensor too large");
    uint32_t fill_bits;
    memcpy(&fill_bits, &fill, 4);
    const bool bfp = dtype == TTMI_BFLOAT8_B || dtype == TTMI_BFLOAT4_B;
    const uint64_t items = bfp ? total / 16 : total;
    const uint32_t blocks = (uint32_t)((items + 255) / 256 < 256 * 32 ? (items + 255) / 256 : 256 * 32);
    switch (dtype) {
        case TTMI_BFLOAT8_B: case TTMI_BFLOAT4_B:
            // whole chunks on both sides (the reference's packers assert it: tt_metal/common/bfloat8.hpp:107)
            if (total % 1024 || src_total % 1024)
                return fail(TTMI_ERR_INVALID_ARGUMENT, "pad / unpad: a block-float tensor holds whole 1024-element chunks (%llu -> %llu elements)",
                            (unsigned long long)src_total, (unsigned long long)total);
            if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u)
                return fail(TTMI_ERR_INVALID_ARGUMENT, "pad / unpad: src and dst must be 16-byte aligned");
            if (dtype == TTMI_BFLOAT8_B) hipLaunchKernelGGL((window_copy_bfp_kernel<7>), dim3(blocks), dim3(256), 0, st, (const uint8_t *)src, (uint8_t *)dst, w, fill_bits, items);
            else hipLaunchKernelGGL((window_copy_bfp_kernel<3>), dim3(blocks), dim3(256), 0, st, (const uint8_t *)src, (uint8_t *)dst, w, fill_bits, items);
            break;
        case TTMI_FLOAT32:
            hipLaunchKernelGGL((window_copy_kernel<uint32_t>), dim3(blocks), dim3(256), 0, st, (const uint32_t *)src, (uint32_t *)dst, w, fill_bits, 1u, items);
            break;
        case TTMI_UINT32:
            hipLaunchKernelGGL((window_copy_kernel<uint32_t>), dim3(blocks), dim3(256), 0, st, (const uint32_t *)src, (uint32_t *)dst, w, (uint32_t)fill, 1u, items);
            break;
        case TTMI_BFLOAT16:      // static_cast<bfloat16>(float) keeps the upper 16 bits (tt_metal/common/bfloat16.hpp:28-38)
            hipLaunchKernelGGL((window_copy_kernel<uint16_t>), dim3(blocks), dim3(256), 0, st, (const uint16_t *)src, (uint16_t *)dst, w, (uint16_t)(fill_bits >> 16), 1u, items);
            break;
        case TTMI_UINT16:
            hipLaunchKernelGGL((window_copy_kernel<uint16_t>), dim3(blocks), dim3(256), 0, st, (const uint16_t *)src, (uint16_t *)dst, w, (uint16_t)fill, 1u, items);
            break;
        default: return fail(TTMI_ERR_INVALID_ARGUMENT, "pad / unpad: unknown dtype %d", dtype);
    }
    return check_launch("window_copy_kernel");
}

// unpad of a TILE-layout tensor at tile granularity: whole tiles are moved, nothing is decoded
int codec_unpad_tiles(uint32_t tile_bytes, const void *src, const uint32_t src_tiles[4], void *dst, const uint32_t start[4],
                      const uint32_t dst_tiles[4], hipStream_t st) {
    WindowDev w{};
    uint64_t total = 1;
    for (int d = 0; d < 4; ++d) {
        if ((uint64_t)start[d] + dst_tiles[d] > src_tiles[d]) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpad: the range leaves the tensor in dimension %d", d);
        w.src[d] = src_tiles[d]; w.dst[d] = dst_tiles[d]; w.off[d] = -(int32_t)start[d];
        total *= dst_tiles[d];
    }
    if (total == 0) return TTMI_OK;
    const uint32_t inner = tile_bytes / 4;
    const uint64_t items = total * inner;
    if (items >> 40) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpad: tensor too large");
    const uint32_t blocks = (uint32_t)((items + 255) / 256 < 256 * 32 ? (items + 255) / 256 : 256 * 32);
    hipLaunchKernelGGL((window_copy_kernel<uint32_t>), dim3(blocks), dim3(256), 0, st, (const uint32_t *)src, (uint32_t *)dst, w, 0u, inner, items);
    return check_launch("window_copy_kernel");
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int W, int ELEM, int MODE, int SHRINK = 0>
static void launch_pack(bool aligned, const void *src, void *dst, const CodecShape &s, uint32_t blocks, hipStream_t st) {
    if (aligned) hipLaunchKernelGGL((pack_kernel<W, ELEM, MODE, true, SHRINK>), dim3(blocks), dim3(256), 0, st, (const uint8_t *)src, (uint8_t *)dst, s);
    else hipLaunchKernelGGL((pack_kernel<W, ELEM, MODE, false, SHRINK>), dim3(blocks), dim3(256), 0, st, (const uint8_t *)src, (uint8_t *)dst, s);
}
template <int W, int ELEM, int MODE, int SHRINK = 0>
static void launch_unpack(bool aligned, const void *src, void *dst, const CodecShape &s, uint32_t blocks, hipStream_t st) {
    if (aligned) hipLaunchKernelGGL((unpack_kernel<W, ELEM, MODE, true, SHRINK>), dim3(blocks), dim3(256), 0, st, (const uint8_t *)src, (uint8_t *)dst, s);
    else hipLaunchKernelGGL((unpack_kernel<W, ELEM, MODE, false, SHRINK>), dim3(blocks), dim3(256), 0, st, (const uint8_t *)src, (uint8_t *)dst, s);
}
// the tensor forms, with the block width chosen for the tensor (tensor_shape)
template <int W, int ELEM>
static void launch_pack_tensor(int shrink, bool aligned, const void *src, void *dst, const CodecShape &s, uint32_t blocks, hipStream_t st) {
    if (shrink == 2) launch_pack<W, ELEM, SRC_TENSOR, 2>(aligned, src, dst, s, blocks, st);
    else if (shrink == 1) launch_pack<W, ELEM, SRC_TENSOR, 1>(aligned, src, dst, s, blocks, st);
    else launch_pack<W, ELEM, SRC_TENSOR, 0>(aligned, src, dst, s, blocks, st);
}
template <int W, int ELEM>
static void launch_unpack_tensor(int shrink, bool aligned, const void *src, void *dst, const CodecShape &s, uint32_t blocks, hipStream_t st) {
    if (shrink == 2) launch_unpack<W, ELEM, SRC_TENSOR, 2>(aligned, src, dst, s, blocks, st);
    else if (shrink == 1) launch_unpack<W, ELEM, SRC_TENSOR, 1>(aligned, src, dst, s, blocks, st);
    else launch_unpack<W, ELEM, SRC_TENSOR, 0>(aligned, src, dst, s, blocks, st);
}

// Blocks of 32 rows x (32 / elem >> shrink) tiles.  Pack and unpack halve the block width (shrink 1, 2) while that is what it
// takes to give the 256 CUs two blocks each: a 1024 x 1024 fp32 tensor is 128 blocks of 8 tiles, but 512 blocks of 2.
static int tensor_shape(CodecShape &s, uint32_t batch, uint32_t h, uint32_t w, size_t row_stride, size_t batch_stride,
                        int elem, uint64_t &blocks, int *shrink = nullptr) {
    s.batch = batch; s.h = h; s.w = w;
    s.ht = (h + 31) / 32; s.wt = (w + 31) / 32;
    uint32_t tpb = 32 / elem;
    s.col_groups = (s.wt + tpb - 1) / tpb;
    if (shrink) {
        *shrink = 0;
        while (*shrink < 2 && (uint64_t)batch * s.ht * s.col_groups < 512 && s.wt > tpb / 2) {
            ++*shrink; tpb /= 2;
            s.col_groups = (s.wt + tpb - 1) / tpb;
        }
    }
    s.n_tiles = (uint64_t)batch * s.ht * s.wt;
    s.row_stride = row_stride; s.batch_stride = batch_stride;
    blocks = (uint64_t)batch * s.ht * s.col_groups;
    if (blocks > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "tensor too large for one launch: %llu blocks", (unsigned long long)blocks);
    return TTMI_OK;
}

int codec_pack_chunks(int fmt, const float *src, size_t n_tiles, int row_major_input, uint32_t *dst, hipStream_t st) {
    if (n_tiles == 0) return TTMI_OK;
    if (!aligned16(src) || !aligned16(dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "pack: src and dst must be 16-byte aligned");
    CodecShape s{};
    s.n_tiles = n_tiles;
    const uint64_t blocks = (n_tiles + 7) / 8;
    if (blocks > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "pack: too many tiles");
    if (fmt == TTMI_BFLOAT8_B) {
        if (row_major_input) launch_pack<7, 4, SRC_TILE_ROWMAJOR>(true, src, dst, s, (uint32_t)blocks, st);
        else launch_pack<7, 4, SRC_TILE_FACES>(true, src, dst, s, (uint32_t)blocks, st);
    } else {
        if (row_major_input) launch_pack<3, 4, SRC_TILE_ROWMAJOR>(true, src, dst, s, (uint32_t)blocks, st);
        else launch_pack<3, 4, SRC_TILE_FACES>(true, src, dst, s, (uint32_t)blocks, st);
    }
    return check_launch("pack_kernel");
}

int codec_unpack_chunks(int fmt, const uint32_t *words, size_t n_tiles, int row_major_output, float *dst, hipStream_t st) {
    if (n_tiles == 0) return TTMI_OK;
    if (!aligned16(words) || !aligned16(dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpack: src and dst must be 16-byte aligned");
    CodecShape s{};
    s.n_tiles = n_tiles;
    const uint64_t blocks = (n_tiles + 7) / 8;
    if (blocks > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpack: too many tiles");
    if (fmt == TTMI_BFLOAT8_B) {
        if (row_major_output) launch_unpack<7, 4, SRC_TILE_ROWMAJOR>(true, words, dst, s, (uint32_t)blocks, st);
        else launch_unpack<7, 4, SRC_TILE_FACES>(true, words, dst, s, (uint32_t)blocks, st);
    } else {
        if (row_major_output) launch_unpack<3, 4, SRC_TILE_ROWMAJOR>(true, words, dst, s, (uint32_t)blocks, st);
        else launch_unpack<3, 4, SRC_TILE_FACES>(true, words, dst, s, (uint32_t)blocks, st);
    }
    return check_launch("unpack_kernel");
}

int codec_pack_tensor(int fmt, const void *src, int elem, uint32_t batch, uint32_t h, uint32_t w, size_t row_stride,
                      size_t batch_stride, uint32_t *dst, hipStream_t st) {
    if ((uint64_t)batch * h * w == 0) return TTMI_OK;
    if (!aligned16(dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "pack: dst must be 16-byte aligned");
    CodecShape s{};
    uint64_t blocks;
    int shrink;
    if (int rc = tensor_shape(s, batch, h, w, row_stride, batch_stride, elem, blocks, &shrink)) return rc;
    const size_t per16 = 16 / elem;
    const bool al = aligned16(src) && w % per16 == 0 && row_stride % per16 == 0 && batch_stride % per16 == 0;
    // every block whole: the straight-line kernel (the bounds of every load and store are those of the tensor itself)
    const bool whole = al && shrink == 0 && h % 32 == 0 && w % (32 * (32 / elem)) == 0;
    if (whole) {
        const dim3 grid((uint32_t)blocks), wg(256);
        if (fmt == TTMI_BFLOAT8_B) {
            if (elem == 4) hipLaunchKernelGGL((pack_whole_kernel<7, 4>), grid, wg, 0, st, (const uint8_t *)src, (uint8_t *)dst, s);
            else hipLaunchKernelGGL((pack_whole_kernel<7, 2>), grid, wg, 0, st, (const uint8_t *)src, (uint8_t *)dst, s);
        } else {
            if (elem == 4) hipLaunchKernelGGL((pack_whole_kernel<3, 4>), grid, wg, 0, st, (const uint8_t *)src, (uint8_t *)dst, s);
            else hipLaunchKernelGGL((pack_whole_kernel<3, 2>), grid, wg, 0, st, (const uint8_t *)src, (uint8_t *)dst, s);
        }
        return check_launch("pack_whole_kernel");
    }
    if (fmt == TTMI_BFLOAT8_B) {
        if (elem == 4) launch_pack_tensor<7, 4>(shrink, al, src, dst, s, (uint32_t)blocks, st);
        else launch_pack_tensor<7, 2>(shrink, al, src, dst, s, (uint32_t)blocks, st);
    } else {
        if (elem == 4) launch_pack_tensor<3, 4>(shrink, al, src, dst, s, (uint32_t)blocks, st);
        else launch_pack_tensor<3, 2>(shrink, al, src, dst, s, (uint32_t)blocks, st);
    }
    return check_launch("pack_kernel");
}

int codec_unpack_tensor(int fmt, const uint32_t *words, uint32_t batch, uint32_t h, uint32_t w, void *dst, int elem,
                        hipStream_t st) {
    if ((uint64_t)batch * h * w == 0) return TTMI_OK;
    if (!aligned16(words)) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpack: words must be 16-byte aligned");
    CodecShape s{};
    uint64_t blocks;
    int shrink;
    if (int rc = tensor_shape(s, batch, h, w, w, (size_t)h * w, elem, blocks, &shrink)) return rc;
    const size_t per16 = 16 / elem;
    const bool al = aligned16(dst) && w % per16 == 0;
    // every block whole: the straight-line kernel (the bounds of every load and store are those of the tensor itself)
    const bool whole = al && shrink == 0 && h % 32 == 0 && w % (32 * (32 / elem)) == 0;
    if (whole) {
        const dim3 grid((uint32_t)blocks), wg(256);
        if (fmt == TTMI_BFLOAT8_B) {
            if (elem == 4) hipLaunchKernelGGL((unpack_whole_kernel<7, 4>), grid, wg, 0, st, (const uint8_t *)words, (uint8_t *)dst, s);
            else hipLaunchKernelGGL((unpack_whole_kernel<7, 2>), grid, wg, 0, st, (const uint8_t *)words, (uint8_t *)dst, s);
        } else {
            if (elem == 4) hipLaunchKernelGGL((unpack_whole_kernel<3, 4>), grid, wg, 0, st, (const uint8_t *)words, (uint8_t *)dst, s);
            else hipLaunchKernelGGL((unpack_whole_kernel<3, 2>), grid, wg, 0, st, (const uint8_t *)words, (uint8_t *)dst, s);
        }
        return check_launch("unpack_whole_kernel");
    }
    if (fmt == TTMI_BFLOAT8_B) {
        if (elem == 4) launch_unpack_tensor<7, 4>(shrink, al, words, dst, s, (uint32_t)blocks, st);
        else launch_unpack_tensor<7, 2>(shrink, al, words, dst, s, (uint32_t)blocks, st);
    } else {
        if (elem == 4) launch_unpack_tensor<3, 4>(shrink, al, words, dst, s, (uint32_t)blocks, st);
        else launch_unpack_tensor<3, 2>(shrink, al, words, dst, s, (uint32_t)blocks, st);
    }
    return check_launch("unpack_kernel");
}

int codec_relayout(bool to_tiles, const void *src, uint32_t elem, uint32_t batch, uint32_t h, uint32_t w, void *dst,
                   hipStream_t st) {
    if ((uint64_t)batch * h * w == 0) return TTMI_OK;
    CodecShape s{};
    uint64_t blocks;
    if (int rc = tensor_shape(s, batch, h, w, w, (size_t)h * w, (int)elem, blocks)) return rc;
    if (!aligned16(to_tiles ? dst : src)) return fail(TTMI_ERR_INVALID_ARGUMENT, "tilize/untilize: the tiled buffer must be 16-byte aligned");
    const size_t per16 = 16 / elem;
    const bool al = aligned16(to_tiles ? src : dst) && w % per16 == 0;
#define TTMI_RELAYOUT(E, T, A) hipLaunchKernelGGL((relayout_kernel<E, T, A>), dim3((uint32_t)blocks), dim3(256), 0, st, (const uint8_t *)src, (uint8_t *)dst, s)
    if (elem == 4) {
        if (to_tiles) { if (al) TTMI_RELAYOUT(4, true, true); else TTMI_RELAYOUT(4, true, false); }
        else { if (al) TTMI_RELAYOUT(4, false, true); else TTMI_RELAYOUT(4, false, false); }
    } else {
        if (to_tiles) { if (al) TTMI_RELAYOUT(2, true, true); else TTMI_RELAYOUT(2, true, false); }
        else { if (al) TTMI_RELAYOUT(2, false, true); else TTMI_RELAYOUT(2, false, false); }
    }
#undef TTMI_RELAYOUT
    return check_launch("relayout_kernel");
}

// bf16 <-> fp32 on flat arrays: fp32 -> bf16 rounds to nearest even, bf16 -> fp32 is exact
template <bool WIDEN>
__global__ __launch_bounds__(256) void convert_float_kernel(const void *__restrict__ src, void *__restrict__ dst, uint64_t count) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (uint64_t)gridDim.x * 256) {
        if (WIDEN) {
            reinterpret_cast<uint32_t *>(dst)[i] = (uint32_t)reinterpret_cast<const uint16_t *>(src)[i] << 16;
        } else {
            typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
            typedef float f32x2_t __attribute__((ext_vector_type(2)));
            const f32x2_t v = {reinterpret_cast<const float *>(src)[i], 0.f};
            reinterpret_cast<uint16_t *>(dst)[i] = (uint16_t)__builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
        }
    }
}

// A tensor in tile order (4-face tiles) from one data type to another, element order unchanged: tt::tt_metal::typecast
// (tt_eager/tt_dnn/op_library/copy/copy_op.hpp:44) for the float formats of this path.  Block-float on either side goes
// through the codec kernels in their face-ordered chunk mode, reading or writing bf16 / fp32 directly.
int codec_typecast_tiles(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n_tiles, hipStream_t st) {
    if (n_tiles == 0) return TTMI_OK;
    const bool src_bfp = src_dtype == TTMI_BFLOAT8_B || src_dtype == TTMI_BFLOAT4_B;
    const bool dst_bfp = dst_dtype == TTMI_BFLOAT8_B || dst_dtype == TTMI_BFLOAT4_B;
    const bool src_float = src_dtype == TTMI_BFLOAT16 || src_dtype == TTMI_FLOAT32;
    const bool dst_float = dst_dtype == TTMI_BFLOAT16 || dst_dtype == TTMI_FLOAT32;
    if (!(src_bfp || src_float) || !(dst_bfp || dst_float) || src_dtype == dst_dtype || (src_bfp && dst_bfp))
        return fail(TTMI_ERR_INVALID_ARGUMENT, "typecast: unsupported conversion %d -> %d", src_dtype, dst_dtype);
    if (!aligned16(src) || !aligned16(dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "typecast: src and dst must be 16-byte aligned");
    CodecShape s{};
    s.n_tiles = n_tiles;
    if (src_bfp || dst_bfp) {
        const int elem = (src_bfp ? dst_dtype : src_dtype) == TTMI_FLOAT32 ? 4 : 2;
        const uint64_t blocks = (n_tiles + (32 / elem) - 1) / (32 / elem);
        if (blocks > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "typecast: too many tiles");
        const int fmt = src_bfp ? src_dtype : dst_dtype;
        if (dst_bfp) {
            if (fmt == TTMI_BFLOAT8_B) { if (elem == 4) launch_pack<7, 4, SRC_TILE_FACES>(true, src, dst, s, (uint32_t)blocks, st); else launch_pack<7, 2, SRC_TILE_FACES>(true, src, dst, s, (uint32_t)blocks, st); }
            else { if (elem == 4) launch_pack<3, 4, SRC_TILE_FACES>(true, src, dst, s, (uint32_t)blocks, st); else launch_pack<3, 2, SRC_TILE_FACES>(true, src, dst, s, (uint32_t)blocks, st); }
            return check_launch("pack_kernel");
        }
        if (fmt == TTMI_BFLOAT8_B) { if (elem == 4) launch_unpack<7, 4, SRC_TILE_FACES>(true, src, dst, s, (uint32_t)blocks, st); else launch_unpack<7, 2, SRC_TILE_FACES>(true, src, dst, s, (uint32_t)blocks, st); }
        else { if (elem == 4) launch_unpack<3, 4, SRC_TILE_FACES>(true, src, dst, s, (uint32_t)blocks, st); else launch_unpack<3, 2, SRC_TILE_FACES>(true, src, dst, s, (uint32_t)blocks, st); }
        return check_launch("unpack_kernel");
    }
    const uint64_t count = (uint64_t)n_tiles * 1024;
    const uint32_t blocks = (uint32_t)((count + 255) / 256 < 256 * 32 ? (count + 255) / 256 : 256 * 32);
    if (src_dtype == TTMI_BFLOAT16) hipLaunchKernelGGL((convert_float_kernel<true>), dim3(blocks), dim3(256), 0, st, src, dst, count);
    else hipLaunchKernelGGL((convert_float_kernel<false>), dim3(blocks), dim3(256), 0, st, src, dst, count);
    return check_launch("convert_float_kernel");
}

}  // namespace ttmi
