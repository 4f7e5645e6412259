// GEMM with block-float weights for gfx950:  C[b,m,n] = act(A[b,m,k] . W[(b|0),k,n] + bias[n]).
//
// Semantics follow tt::operations::primary::matmul (tt_eager/tt_dnn/op_library/bmm/bmm_op.hpp:318-346,
// bmm_op.cpp:828-1049): bf16 activations, BFLOAT8_B / BFLOAT4_B weights stored as packed 32x32 tiles
// (tile (kt, nt) at index kt*Nt + nt; layout of one tile: tt_metal/common/bfloat8.hpp:102-173), fp32
// accumulation, bf16 (or fp32) output.  Weight values are what the reference unpacker produces
// (bfloat8.hpp:229-249, tt_metal/common/bfloat4.hpp:113-146): sign * mantissa * 2^(E - 127 - (W-1)); they
// carry at most 7 significant bits, so the conversion to bf16 in front of the matrix cores is exact.
//
// Streaming kernel (weights are read from HBM once per 32-row band of A; decode shapes are HBM-bound):
//   unit       one k-tile (32 rows of W) of one output group; an output group is a 32-row band of one batch slice
//              times 64 columns (2 adjacent packed tiles, one contiguous run in memory)
//   wavefront  brings the 2 tiles of a unit into its private LDS ring with direct global->LDS loads (no staging
//              registers), units ahead of the arithmetic; per unit it builds four pairs of B operands in hidden-one form
//              (bfp_dequant.h: no conversion, no multiplication) and issues sixteen v_mfma_f32_16x16x32_bf16.  Lane
//              (c, g) — c = lane % 16, g = lane / 16 — holds, for operand j, column 4c+j of the group and k rows
//              8g..8g+7: byte j of the 8 mantissa words it reads from LDS.  The packed layout (16 consecutive columns of
//              one k row share a word run) never has to be transposed.
//   workgroup  4 wavefronts take the units of a contiguous range round-robin, add their partial sums through LDS
//              and store; the range is one of the nearly equal parts the host cuts every output's k range into, as
//              many as fill the chip.  Outputs whose k range is shared between workgroups are finished by the
//              workgroup that owns the last part (see the kernel).
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cmath>
#include <stdint.h>
#include <mutex>
#include <type_traits>
#include <utility>

#include "bfp_dequant.h"
#include "ttmi_internal.h"

namespace ttmi {

// n / d for a divisor known on the host and any n < 2^31, without a division on the device (a 32-bit division is some forty
// instructions in a dependent chain, and the kernels below divide before they can request their first byte):
// with s = ceil(log2 d) and M = ceil(2^(32+s) / d) = 2^32 + mul, n / d = (mulhi(n, mul) + n) >> s.
struct FastDiv {
    uint32_t mul, shift;
    __host__ __device__ __forceinline__ uint32_t operator()(uint32_t n) const {
#if defined(__HIP_DEVICE_COMPILE__)
        return (__umulhi(n, mul) + n) >> shift;
#else
        return (uint32_t)((((uint64_t)n * mul) >> 32) + n) >> shift;
#endif
    }
};
inline FastDiv fast_div(uint32_t d) {
    FastDiv f{0, 0};
    if (d <= 1) return f;
    uint32_t s = 0;
    while ((1ull << s) < d) ++s;
    const unsigned __int128 one = 1;
    const unsigned __int128 m = ((one << (32 + s)) + d - 1) / d;
    f.mul = (uint32_t)(m - (one << 32));
    f.shift = s;
    return f;
}

struct MatmulDev {
    const uint8_t *a;        // bf16
    const uint8_t *b;        // packed tiles
    const uint8_t *b2;       // gated form only: the second weight matrix (same shape and format), C = act(A.b) * (A.b2)
    const uint16_t *bias;    // bf16 [n] or null
    uint8_t *c;              // output (bf16 or fp32)
    float *slots;            // 2 slots of 32x64 fp32 per workgroup, for outputs shared between workgroups (see SLOT_EMPTY)
    uint32_t *error;         // the device's error word (host memory): raised when a wait for partial sums gives up
    uint32_t spin_limit;     // polls before such a wait gives up
    int drop_partial_sums;   // test only: producers keep their sums to themselves, so that the wait must give up
    uint32_t batch, b_batch, m, k, n;
    uint32_t mt, kt, nt, ngroups;
    uint32_t mt_sets;        // 128-column kernel: sets of row bands that share a workgroup (mt, or ceil(mt / 2) in the two-band form)
    uint32_t groups;         // batch * mt * ngroups
    uint32_t workgroups;     // P
    uint32_t units;          // U = batch * mt * ngroups * kt
    uint32_t split;          // k ranges per output group (>= 1)
    FastDiv by_split, by_ngroups, by_mt_sets;     // 128-column kernel: divisions by split, ngroups and mt_sets
    uint32_t xcds;           // 128-column kernel: 8 when workgroups b and b + 8 are known to run on one XCD (the workgroups that share an output are then placed there), else 1
    int a_tiled, c_tiled, c_f32;
    int c_bfp;               // 128-column kernel only: 0, or the mantissa bits (7 | 3) of a block-float output in TILE layout
};

constexpr int GROUP_TILES = 2;                       // n tiles per output group
constexpr int GROUP_COLS = GROUP_TILES * 32;
constexpr int WAVES = 4;
#ifndef TTMI_STREAM_WGS_PER_CU
#define TTMI_STREAM_WGS_PER_CU 3
#endif
#ifndef TTMI_STREAM_STAGES
#define TTMI_STREAM_STAGES 3
#endif
constexpr int WGS_PER_CU = TTMI_STREAM_WGS_PER_CU;   // workgroups of 4 wavefronts per CU (registers and LDS allow 3)
constexpr int STAGES = TTMI_STREAM_STAGES;           // LDS ring per wavefront = units requested ahead of the arithmetic
constexpr int A_LOADS = 2;                           // activation loads per unit (rows c and c + 16 of the band)
constexpr int REDUCE_BYTES = WAVES * 32 * 64 * 4;    // every wavefront lays out its 32 accumulator registers
constexpr size_t SLOT_BYTES = 32 * GROUP_COLS * sizeof(float);

// Partial sums that other workgroups read travel through device-coherent accesses (the sc1 bit: past the per-XCD L2,
// which is not coherent across XCDs), 16 bytes per lane, so neither a cache write-back nor an invalidate is needed —
// a full agent-scope fence here costs more than the whole GEMM.  There are no flags and no counters: every slot
// word holds SLOT_EMPTY between launches, the producer overwrites it with data (which it keeps from ever having
// that bit pattern), and the consumer simply re-reads until no word is SLOT_EMPTY, then puts SLOT_EMPTY back.
constexpr uint32_t SLOT_EMPTY = 0xffffffffu;         // a NaN that arithmetic on bf16-derived inputs does not produce
constexpr uint32_t SLOT_SPIN_LIMIT = 1u << 20;       // bounded wait: a lost producer must not hang the GPU
constexpr uint32_t ERROR_SLOT_TIMEOUT = 1;           // what the error word is set to

// A wait that gave up: tell the host (one plain store into the error word, which lives in host memory) and carry on,
// so that the grid still drains.  The output of this launch is invalid and the call that follows reports it.
__device__ __forceinline__ void report_timeout(const MatmulDev &p) {
    if ((threadIdx.x & 63) == 0) __builtin_nontemporal_store(ERROR_SLOT_TIMEOUT, p.error);
}

__device__ __forceinline__ void slot_store(float4 *to, const u32x4 v) {
    // A store of more than 8 bytes reads its data registers for two more cycles after it has issued; the compiler
    // inserts the wait states for stores of its own, here the s_nop does it.
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(to), "v"(v) : "memory");
}
// The same for a reader in the writer's own XCD: the vector L1 writes through, so a plain store puts the data into the
// XCD's L2, which all its CUs share, and a device-scope load (slot_load_issue) finds it there.  Measured with two
// workgroups passing a word back and forth: 0.52 us per round trip against 0.78 us with device-scope stores (0.84 us
// between XCDs); loads of any narrower scope are served from the reader's vector L1 when a line is read a second time.
__device__ __forceinline__ void slot_store_same_xcd(float4 *to, const u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" ::"v"(to), "v"(v) : "memory");
}

__device__ __forceinline__ u32x4 slot_load_issue(const float4 *from) {
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(from) : "memory");
    return v;
}
__device__ __forceinline__ uint32_t not_empty(uint32_t bits) { return bits == SLOT_EMPTY ? 0xfffffffeu : bits; }

// Which units a workgroup takes: every output group is cut into `split` nearly equal k ranges, one per workgroup
// (P = groups * split): one output per workgroup, at most `split` partial sums to add.  Units are numbered with the
// k-tile fastest.
__host__ __device__ __forceinline__ uint32_t range_start(uint32_t kt, uint32_t split, uint32_t i) {
    return (i / split) * kt + ((i % split) * kt) / split;
}
__host__ __device__ __forceinline__ uint32_t workgroup_of(uint32_t kt, uint32_t split, uint32_t unit) {
    const uint32_t og = unit / kt, within = unit - og * kt;
    return og * split + ((within + 1) * split - 1) / kt;     // largest part j with (j * kt) / split <= within
}
__device__ __forceinline__ uint32_t range_start(const MatmulDev &p, uint32_t i) { return range_start(p.kt, p.split, i); }
__device__ __forceinline__ uint32_t workgroup_of(const MatmulDev &p, uint32_t unit) { return workgroup_of(p.kt, p.split, unit); }

// Work decomposition: units are numbered with the k-tile fastest; a workgroup takes a contiguous range of them (see
// range_start).  A workgroup whose range covers all k-tiles of an output group stores that output directly.
// Otherwise the contributors to an output hand their fp32 partial sums over in slots: every contributor but the one
// with the highest index writes its sums to its own slot; that last one waits for each slot to lose its SLOT_EMPTY
// pattern, adds the slots in workgroup order to its own sums (so the result does not depend on timing), applies the
// epilogue, stores, and puts the empty pattern back.
// every word of a caller's workspace becomes SLOT_EMPTY
__global__ __launch_bounds__(256) void fill_slots_kernel(u32x4 *slots, uint32_t chunks) {
    const u32x4 empty = {SLOT_EMPTY, SLOT_EMPTY, SLOT_EMPTY, SLOT_EMPTY};
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < chunks; i += gridDim.x * 256) slots[i] = empty;
}

template <int... Is, typename Fn> __device__ __forceinline__ void static_for(std::integer_sequence<int, Is...>, Fn fn) {
    (fn(std::integral_constant<int, Is>{}), ...);
}
// step(J) for J = FROM, FROM + 1, ... while first + J < total and J < COUNT
template <int FROM, int COUNT, typename Step> __device__ __forceinline__ void nested_steps(uint32_t first, uint32_t total, Step step) {
    if constexpr (FROM < COUNT) {
        if (first + FROM < total) {
            step(std::integral_constant<int, FROM>{});
            nested_steps<FROM + 1, COUNT>(first, total, step);
        }
    }
}
// waits until at most min(younger, MOST) * PER requests are in flight
template <int MOST, int PER> __device__ __forceinline__ void wait_for_younger(uint32_t younger) {
    if constexpr (MOST == 0) {
        wait_vmcnt<0>();
    } else {
        if (younger >= (uint32_t)MOST) wait_vmcnt<MOST * PER>(); else wait_for_younger<MOST - 1, PER>(younger);
    }
}

template <int W, int ACT>
__global__ __launch_bounds__(256, WGS_PER_CU) void matmul_stream_kernel(const MatmulDev p) {
    using F = Wfmt<W>;
    constexpr int WAVE_LDS = STAGES * F::stage_bytes;
    constexpr int LDS_BYTES = REDUCE_BYTES > WAVES * WAVE_LDS ? REDUCE_BYTES : WAVES * WAVE_LDS;
    constexpr int NLOAD = F::loads;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[LDS_BYTES];

    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;                      // column quad and k-row group of this lane
    const int t_of_lane = c >> 3, fc = (c >> 2) & 1, q = c & 3;  // tile, face column and word inside the face row
    const int h_of_lane = g >> 1, g_low = g & 1;                 // k rows 8g..8g+7 = rows 8*g_low.. of face 2*h + fc

    // ---- addressing that does not depend on the segment ---------------------------------------------------
    uint32_t chunk_of[NLOAD];
    stage_chunks<W>(lane, chunk_of);
    // per-lane LDS offsets inside a stage (offsets, not pointers: the accesses stay LDS instructions)
    const uint32_t exp_off = wave * WAVE_LDS + F::exp_base + t_of_lane * 64 + (2 * h_of_lane + fc) * 16 + g_low * 8;
    const uint32_t mant_off = wave * WAVE_LDS + (h_of_lane * 4 + t_of_lane * 2 + fc) * F::face_stride + (g_low * 8) * F::row_bytes +
                              (W == 7 ? q * 4 : (q >> 1) * 4);
    const uint64_t w_step = (uint64_t)WAVES * p.nt * F::tile_bytes;      // bytes between the units of one wavefront
    const uint32_t a_step = p.a_tiled ? WAVES * 2048 : WAVES * 64;

    f32x4 acc[2][4];                                  // [16-row half of the band][operand j]
    u32x4 a_ring[STAGES][2] = {};                     // activations of the units in flight, one entry per LDS stage
    uint32_t src_off[NLOAD];
    uint32_t a_half = 0;                              // bytes from row c to row c + 16 of the band (set per segment)
    const uint8_t *wptr = nullptr, *aptr = nullptr;

    // Requests one unit: its 2 packed tiles straight into LDS stage S, its activations into a_ring[S].
    auto fetch = [&](auto stage_tag) __attribute__((always_inline)) {
        constexpr int S = decltype(stage_tag)::value;
#pragma unroll
        for (int l = 0; l < NLOAD; ++l)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(wptr + src_off[l]),
                                             (__attribute__((address_space(3))) void *)(lds + wave * WAVE_LDS + S * F::stage_bytes + l * 1024),
                                             16, 0, 0);
        wptr += w_step;
        // The activation loads and the waits for them are inline assembly as well: with direct-to-LDS loads pending
        // the compiler waits for ALL vector-memory operations before the first use of any loaded register.  The
        // ring registers are read-write operands, so each entry stays in one physical register from request to use.
        asm volatile("global_load_dwordx4 %0, %1, off" : "+v"(a_ring[S][0]) : "v"(aptr) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off" : "+v"(a_ring[S][1]) : "v"(aptr + a_half) : "memory");
        aptr += a_step;
    };
    // Works on the unit in stage S; once its LDS reads have returned the stage is handed to unit i + STAGES.
    // `younger` = units requested after this one and still allowed to be in flight.
    auto work = [&](auto stage_tag, auto younger_tag, bool refill) __attribute__((always_inline)) {
        constexpr int S = decltype(stage_tag)::value;
        constexpr int YOUNGER = decltype(younger_tag)::value;
        if (YOUNGER >= 0) wait_vmcnt<(YOUNGER < 0 ? 0 : YOUNGER) * (NLOAD + A_LOADS)>();   // < 0: the caller has waited
        asm volatile("" : "+v"(a_ring[S][0]), "+v"(a_ring[S][1]) :: "memory");          // uses stay behind the wait
        // The activations leave the ring through explicit moves: the ring registers are then free for the next
        // request, which lands in them directly (a copy of a register still being loaded would wait for the load).
        u32x4 a_now[2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint32_t moved;
                asm volatile("v_mov_b32 %0, %1" : "=v"(moved) : "v"(a_ring[S][h][e]));
                a_now[h][e] = moved;
            }
        // weights in hidden-one form (bfp_dequant.h): A.W = 2 (A.hi - A.lo), the subtraction as an MFMA with the negated activations
        u32x4 a_neg[2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) a_neg[h][e] = a_now[h][e] ^ 0x80008000u;
        SlabRaw raw;
        slab_read<W, S * F::stage_bytes, S * F::stage_bytes>(lds_base + exp_off, lds_base + mant_off, raw);
        wait_slab(raw);
        if (refill) fetch(stage_tag);
        bf16x8 hi[4], lo[4];
        slab_expand_hidden<W>(raw, q, hi, lo);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[h][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a_now[h]), hi[j], acc[h][j], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[h][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a_neg[h]), lo[j], acc[h][j], 0, 0, 0);
        }
    };

    const uint32_t me = blockIdx.x;
    uint32_t unit = range_start(p, me);
    const uint32_t unit_end = range_start(p, me + 1);
    const uint32_t my_first_og = unit / p.kt;

    while (unit < unit_end) {
        // ---- one segment: output group og, k-tiles [k_begin, k_end) ---------------------------------------
        const uint32_t og = unit / p.kt;
        const uint32_t k_begin = unit - og * p.kt;
        const uint32_t k_end = min(p.kt, k_begin + (unit_end - unit));
        unit += k_end - k_begin;
        const uint32_t ng = og % p.ngroups, band = og / p.ngroups;
        const uint32_t mt = band % p.mt, bb = band / p.mt;
        const uint32_t nt0 = ng * GROUP_TILES;
        const uint32_t n_valid = min((uint32_t)GROUP_TILES, p.nt - nt0);

        // tiles past the matrix edge repeat the last chunk that exists and are never stored
        const uint32_t chunks_valid = n_valid * F::chunks;
#pragma unroll
        for (int l = 0; l < NLOAD; ++l) src_off[l] = min(chunk_of[l], chunks_valid - 1) * 16;
        wptr = p.b + ((uint64_t)(p.b_batch == 1 ? 0 : bb) * p.kt * p.nt + (uint64_t)(k_begin + wave) * p.nt + nt0) * F::tile_bytes;
        // activations of one unit for this lane: rows c and c + 16 of the band, k = kt*32 + 8g .. 8g + 7;
        // rows past M read row M-1 and are never stored
        if (p.a_tiled) {
            aptr = p.a + (((uint64_t)bb * p.mt + mt) * p.kt + k_begin + wave) * 2048 + h_of_lane * 512 + c * 32 + g_low * 16;
            a_half = 1024;
        } else {
            const uint32_t r0 = min(mt * 32 + c, p.m - 1), r1 = min(mt * 32 + c + 16, p.m - 1);
            aptr = p.a + (((uint64_t)bb * p.m + r0) * p.k + (k_begin + wave) * 32 + g * 8) * 2;
            a_half = (r1 - r0) * p.k * 2;
        }

#pragma unroll
        for (int mh = 0; mh < 2; ++mh)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[mh][j][r] = 0.f;

        // This wavefront's units: k_begin + wave, + WAVES, ... (`total` of them).  Unit i lives in stage i % STAGES and
        // is requested STAGES units ahead: when unit i has been read out of its stage, unit i + STAGES is requested
        // into it.  Vector-memory operations complete in order, so at the top of unit i exactly the requests of the
        // units after it may still be in flight: min(STAGES - 1, total - 1 - i) of them.
        const uint32_t span = k_end - k_begin;
        const uint32_t total = span > (uint32_t)wave ? (span - wave + WAVES - 1) / WAVES : 0;
        using Last = std::integral_constant<int, STAGES - 1>;
        constexpr auto stages = std::make_integer_sequence<int, STAGES>{};
        uint32_t i = 0;
        if (total >= 2 * STAGES) {
            // steady state: every unit worked on here has a successor to request, so the number of requests in
            // flight at each wait is a constant the compiler can see (no conditional request on the way in)
            static_for(stages, [&](auto s) __attribute__((always_inline)) { fetch(s); });
#pragma unroll 1
            for (; i + 2 * STAGES <= total; i += STAGES)
                static_for(stages, [&](auto s) __attribute__((always_inline)) { work(s, Last{}, true); });
        } else {
            static_for(stages, [&](auto s) __attribute__((always_inline)) { if (total > (uint32_t)decltype(s)::value) fetch(s); });
        }
        // at most 2 * STAGES - 1 units are left, starting in stage 0
        static_for(std::make_integer_sequence<int, 2 * STAGES - 1>{}, [&](auto j) __attribute__((always_inline)) {
            constexpr int J = decltype(j)::value;
            const uint32_t at = i + J;
            if (at >= total) return;
            wait_for_younger<STAGES - 1, NLOAD + A_LOADS>(total - 1 - at);
            // a unit requested from here would be number J + STAGES of the tail: only the first STAGES - 1 steps can have one
            work(std::integral_constant<int, J % STAGES>{}, std::integral_constant<int, -1>{}, J + STAGES < 2 * STAGES - 1 && at + STAGES < total);
        });

        wait_vmcnt<0>();   // nothing in flight any more (already true; also what the build-time ISA check keys on)
        // ---- add the four wavefronts' partial sums through LDS --------------------------------------------------
        // Every wavefront writes all 32 of its accumulator registers (register indices are compile-time constants;
        // who reads what is decided by addresses), then wavefront w keeps half w/2 of the band, registers
        // 2*(w%2) and 2*(w%2)+1: rows (w/2)*16 + 4g + 2*(w%2) + {0, 1}, all 64 columns.
        __syncthreads();
        float *red = reinterpret_cast<float *>(lds);
#pragma unroll
        for (int mh = 0; mh < 2; ++mh)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) red[(wave * 32 + mh * 16 + j * 4 + r) * 64 + lane] = acc[mh][j][r];
        __syncthreads();
        float mine[2][4];   // [r][j]
        {
            const float *from = red + ((wave >> 1) * 16 + (wave & 1) * 2) * 64 + lane;
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float v = 0.f;
#pragma unroll
                    for (int sw = 0; sw < WAVES; ++sw) v += from[(sw * 32 + j * 4 + r) * 64];
                    mine[r][j] = v;
                }
        }

        // ---- outputs shared with other workgroups ----------------------------------------------------------
        // Contributors are the workgroups first..last whose ranges meet this output's k range.  The last one (the
        // highest index: every other contributor was dispatched before it and waits for nobody, so it will finish)
        // collects the others' partial sums and adds them in workgroup order, its own last: the result does not
        // depend on timing.  Wavefront w of every contributor holds the same rows, so the hand-over is wavefront to
        // wavefront and needs no workgroup barrier.
        bool store_now = true;
        if (k_begin != 0 || k_end != p.kt) {
            const uint32_t lo = og * p.kt;
            const uint32_t first = workgroup_of(p, lo), last = workgroup_of(p, lo + p.kt - 1);
            if (me != last) {
                float4 *slot = reinterpret_cast<float4 *>(p.slots) + ((uint64_t)(2 * me + (og == my_first_og ? 0 : 1)) * 8 + wave * 2) * 64 + lane;
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    u32x4 v;
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = not_empty(__float_as_uint(mine[r][j]));
                    if (!p.drop_partial_sums) slot_store(slot + r * 64, v);
                }
                store_now = false;
            } else {
                float sum[2][4];
#pragma unroll
                for (int r = 0; r < 2; ++r)
#pragma unroll
                    for (int j = 0; j < 4; ++j) sum[r][j] = 0.f;
                const u32x4 empty = {SLOT_EMPTY, SLOT_EMPTY, SLOT_EMPTY, SLOT_EMPTY};
                for (uint32_t w0 = first; w0 < last; w0 += 4) {          // four contributors' loads in flight at a time
                    u32x4 part[4][2];
                    float4 *other[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const uint32_t w = min(w0 + u, last - 1);
                        const uint32_t which = range_start(p, w) >= lo ? 0u : 1u;      // first or second output of w
                        other[u] = reinterpret_cast<float4 *>(p.slots) + ((uint64_t)(2 * w + which) * 8 + wave * 2) * 64 + lane;
                    }
                    uint32_t spins = 0;
                    bool waiting;
                    do {
#pragma unroll
                        for (int u = 0; u < 4; ++u)
#pragma unroll
                            for (int r = 0; r < 2; ++r) part[u][r] = slot_load_issue(other[u] + r * 64);
                        asm volatile("s_waitcnt vmcnt(0)" : "+v"(part[0][0]), "+v"(part[0][1]), "+v"(part[1][0]), "+v"(part[1][1]),
                                     "+v"(part[2][0]), "+v"(part[2][1]), "+v"(part[3][0]), "+v"(part[3][1])::"memory");
                        bool missing = false;
#pragma unroll
                        for (int u = 0; u < 4; ++u)
#pragma unroll
                            for (int r = 0; r < 2; ++r)
#pragma unroll
                                for (int j = 0; j < 4; ++j) missing |= part[u][r][j] == SLOT_EMPTY;
                        const bool any_missing = __ballot(missing) != 0;
                        waiting = any_missing && ++spins < p.spin_limit;
                        if (waiting) __builtin_amdgcn_s_sleep(4);
                        else if (any_missing) report_timeout(p);
                    } while (waiting);
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (w0 + u >= last) break;
#pragma unroll
                        for (int r = 0; r < 2; ++r) {
#pragma unroll
                            for (int j = 0; j < 4; ++j) sum[r][j] += __uint_as_float(part[u][r][j]);
                            slot_store(other[u] + r * 64, empty);                       // ready for the next launch
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < 2; ++r)
#pragma unroll
                    for (int j = 0; j < 4; ++j) mine[r][j] = sum[r][j] + mine[r][j];
            }
        }

        if (store_now && t_of_lane < (int)n_valid) {
            const uint32_t n_col = (nt0 + t_of_lane) * 32 + fc * 16 + q * 4;   // first of this lane's 4 columns
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const uint32_t row_in_band = (wave >> 1) * 16 + g * 4 + (wave & 1) * 2 + r;
                const uint32_t row = mt * 32 + row_in_band;
                if (row >= p.m) continue;
                float v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float x = mine[r][j] * hidden_unscale;
                    if (p.bias) x += __uint_as_float((uint32_t)p.bias[n_col + j] << 16);
                    v[j] = apply_activation<ACT>(x);
                }
                uint64_t elem;   // element offset of the 4-column run in C
                if (p.c_tiled) {
                    const uint64_t tile = ((uint64_t)bb * p.mt + mt) * p.nt + nt0 + t_of_lane;
                    elem = tile * 1024 + ((row_in_band >> 4) * 2 + fc) * 256 + (row_in_band & 15) * 16 + q * 4;
                } else {
                    elem = ((uint64_t)bb * p.m + row) * p.n + n_col;
                }
                if (p.c_f32) {
                    *reinterpret_cast<float4 *>(p.c + elem * 4) = make_float4(v[0], v[1], v[2], v[3]);
                } else {
                    const uint32_t lo16 = f32x2_to_bf16x2_rne(v[0], v[1]);
                    const uint32_t hi16 = f32x2_to_bf16x2_rne(v[2], v[3]);
                    *reinterpret_cast<uint2 *>(p.c + elem * 2) = make_uint2(lo16, hi16);
                }
            }
        }
        __syncthreads();   // LDS is reused by the next segment
    }
}

// ---------------------------------------------------------------------------------------------------------
// Wide streaming kernel: the same scheme with units of 32 k rows x 128 columns (4 adjacent packed tiles) and
// v_mfma_f32_32x32x16_bf16.  Against the 64-column kernel every activation load, every ring move and every matrix
// instruction serves twice as many weights.
//   lane (c32 = lane % 32, kh = lane / 32) holds, for operand j of slab s (k rows 16s..16s+15 of the k-tile),
//   column 4*c32 + j of the group and k rows 16s + 8kh .. + 7: byte j of 8 mantissa words of face row s of tile
//   c32 / 8.  The activations are the A operand of the same instruction: row c32 of the band, the same 8 k.
//   One workgroup = one k range of one output group (split >= 1); after the loop acc[j][i] is row 8(i/4) + 4kh + i%4,
//   column 4*c32 + j.  Wavefront w keeps rows 8w..8w+7 of the workgroup's sums.
// A stage of the LDS ring holds the four tiles of a unit as WideFmt describes (bfp_dequant.h): as they lie in memory,
// fetched so that four neighbouring lanes ask for one aligned 64-byte piece, and placed so that the 64 lanes of one
// ds_read2_b32 fall into 64 different banks.
// ---------------------------------------------------------------------------------------------------------
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
constexpr int WIDE_TILES = 4;
constexpr int WIDE_COLS = WIDE_TILES * 32;
#ifndef TTMI_WIDE_WGS_PER_CU
#define TTMI_WIDE_WGS_PER_CU 2
#endif
#ifndef TTMI_WIDE_STAGES
#define TTMI_WIDE_STAGES 2      // measured: 2 beats 3 by 1.5 us on the Falcon h_to_4h shape (less code, fewer registers), 4 leaves one workgroup per CU
#endif
constexpr int WEIGHTS_ONCE = 2;     // cache policy of the weight loads: nt (read once, not to displace the activations in L2); measured 0.4 us per launch
constexpr int WIDE_WGS_PER_CU = TTMI_WIDE_WGS_PER_CU;
constexpr int WIDE_STAGES = TTMI_WIDE_STAGES;
constexpr int WIDE_REDUCE_BYTES = WAVES * 64 * 64 * 4;     // every wavefront lays out the 64 accumulator registers of one set of sums
constexpr size_t WIDE_SLOT_BYTES = 32 * WIDE_COLS * sizeof(float);

// NB = 2 is the gated form, C = act(A . B) * (A . B2) (silu(x w1) * (x w3) of a gated MLP in one launch): a unit is then
// the same k-tile and column group of both weight matrices, which share the activations; every workgroup keeps two sets
// of sums and hands over two slots.
// MB = 2 is the two-band form for 33 to 127 rows: a unit is one k-tile and column group of the weights against two
// 32-row bands of the activations, so that the weights are streamed once per 64 rows.  Either way a workgroup keeps
// X = NB * MB sets of sums (one of NB, MB is 1).
// 128-column kernel with the output groups dealt out to 8 XCDs: the number (group * split + part) of the workgroup with
// hardware index b, which runs on XCD (b + c) % 8 and is number b / 8 there: group (b / 8 / split) * 8 + b % 8
__host__ __device__ __forceinline__ uint32_t wide_workgroup_number(uint32_t b, uint32_t split, FastDiv by_split) {
    const uint32_t in_xcd = b >> 3, local_group = by_split(in_xcd);
    return (local_group * 8 + (b & 7)) * split + (in_xcd - local_group * split);
}

template <int W, int ACT, int NB, int MB, bool A8 = false>
__global__ __launch_bounds__(256, NB == 2 ? 1 : WIDE_WGS_PER_CU) void matmul_wide_kernel(const MatmulDev p) {
    using F = WideFmt<W>;
    constexpr int X = NB * MB;
    static_assert(X <= 2, "one of NB, MB is 1");
    static_assert(!A8 || NB == 1, "block-float activations: one weight matrix");
    constexpr int UNIT_BYTES = NB * F::unit_bytes;     // a stage holds the unit's tiles of every weight matrix
    constexpr int WAVE_LDS = WIDE_STAGES * UNIT_BYTES;
    constexpr int LDS_BYTES = WIDE_REDUCE_BYTES > WAVES * WAVE_LDS ? WIDE_REDUCE_BYTES : WAVES * WAVE_LDS;
    constexpr int NLOAD = F::loads;
    constexpr int PER = NB * NLOAD + (A8 ? 4 : 2) * MB;   // vector-memory requests per unit
    __shared__ __attribute__((aligned(1024))) uint8_t lds[LDS_BYTES];

    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // scalar: branches on it are uniform
    const int c32 = lane & 31, kh = lane >> 5;
    const int t_of_lane = c32 >> 3, fc = (c32 >> 2) & 1, q = c32 & 3;

    uint32_t chunk_of[NLOAD];
    wide_stage_chunks<W>(lane, chunk_of);
    // this lane's LDS addresses for slab 0 of stage 0; slab 1 is 32 bytes (exponents) / F::slab_bytes (mantissas) further
    const uint32_t exp_at = lds_base + wave * WAVE_LDS + wide_exp_at<W>(t_of_lane, fc, kh);
    const uint32_t mant_at = lds_base + wave * WAVE_LDS + wide_mant_at<W>(t_of_lane, fc, q, kh);

    // ---- this workgroup's output group and k range ---------------------------------------------------------
    // Output groups are dealt out to the XCDs in turn and the workgroups of a group are consecutive inside their XCD: the
    // hardware's dispatcher hands consecutive workgroups of a launch to consecutive XCDs, so workgroups b and b + 8 run on
    // the same one (whichever it is: the first workgroup's XCD differs from queue to queue) and the partial sums of an
    // output never leave the L2 of one XCD.  Were the placement ever different, a collector would not see sums that sit in
    // another XCD's L2: its bounded wait gives up and the launch is reported, it does not return wrong sums.  `me` numbers
    // the workgroups group by group; slots and waits below are told in terms of it.
    const bool in_xcds = p.xcds == 8;
    const uint32_t me = in_xcds ? wide_workgroup_number(blockIdx.x, p.split, p.by_split) : blockIdx.x;
    const uint32_t before = in_xcds ? 8 : 1;           // the output group that this workgroup's group collects lies this far back
    const uint32_t og = p.by_split(me), part = me - og * p.split;
    const uint32_t k_begin = p.by_split(part * p.kt), k_end = p.by_split((part + 1) * p.kt);
    const uint32_t band = p.by_ngroups(og), ng = og - band * p.ngroups;
    const uint32_t bb = p.by_mt_sets(band), mt = (band - bb * p.mt_sets) * MB;       // batch slice, first row band of this workgroup
    const uint32_t nt0 = ng * WIDE_TILES;
    const uint32_t n_valid = min((uint32_t)WIDE_TILES, p.nt - nt0);

    // tiles past the matrix edge repeat the last chunk that exists and are never stored
    const uint32_t chunks_valid = n_valid * F::chunks;
    uint32_t src_off[NLOAD];
#pragma unroll
    for (int l = 0; l < NLOAD; ++l) src_off[l] = min(chunk_of[l], chunks_valid - 1) * 16;
    const uint64_t w_first = ((uint64_t)(p.b_batch == 1 ? 0 : bb) * p.kt * p.nt + (uint64_t)(k_begin + wave) * p.nt + nt0) * F::tile_bytes;
    const uint8_t *wptr[NB];
    wptr[0] = p.b + w_first;
    if (NB == 2) wptr[NB - 1] = p.b2 + w_first;
    const uint64_t w_step = (uint64_t)WAVES * p.nt * F::tile_bytes;
    // activations of one unit for this lane: row c32 of the band, k = kt*32 + 16s + 8kh .. + 7 for s = 0, 1;
    // rows past M read row M-1 and are never stored
    // (a second band past the last one repeats the last one and is never stored)
    // Block-float activations (A8: packed BFLOAT8_B tiles): the lane's 8 codes are half of a 16-byte face row — face
    // 2 (c32 / 16) + s of the tile, row c32 % 16 — which both lanes of the row load whole, and the row's exponent byte
    // comes by a load of its own (eptr).
    const uint8_t *aptr[MB], *eptr[MB];
    uint32_t a_second, a_step;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const uint32_t band_mt = min(mt + mb, p.mt - 1);
        eptr[mb] = nullptr;
        if (A8) {
            const uint8_t *tile = p.a + (((uint64_t)bb * p.mt + band_mt) * p.kt + k_begin + wave) * 1088;
            aptr[mb] = tile + 64 + (c32 >> 4) * 512 + (c32 & 15) * 16;
            eptr[mb] = tile + (c32 >> 4) * 32 + (c32 & 15);
        } else if (p.a_tiled) {
            aptr[mb] = p.a + (((uint64_t)bb * p.mt + band_mt) * p.kt + k_begin + wave) * 2048 + (c32 >> 4) * 1024 + (c32 & 15) * 32 + kh * 16;
        } else {
            const uint32_t r0 = min(band_mt * 32 + c32, p.m - 1);
            aptr[mb] = p.a + (((uint64_t)bb * p.m + r0) * p.k + (k_begin + wave) * 32 + kh * 8) * 2;
        }
    }
    if (A8) { a_second = 256; a_step = WAVES * 1088; } else if (p.a_tiled) { a_second = 512; a_step = WAVES * 2048; } else { a_second = 32; a_step = WAVES * 64; }

    f32x16 acc[X][4];
#pragma unroll
    for (int x = 0; x < X; ++x)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[x][j][i] = 0.f;
    // The ring registers are cleared by instructions the compiler cannot see through: entries it knows to be zero it
    // would keep in a shared constant register and copy loaded entries around at joins, while their loads are in flight.
    u32x4 a_ring[WIDE_STAGES][2 * MB];                  // [stage][2 * band + slab]
#pragma unroll
    for (int s = 0; s < WIDE_STAGES; ++s)
#pragma unroll
        for (int h = 0; h < 2 * MB; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint32_t zero;
                asm volatile("v_mov_b32 %0, 0" : "=v"(zero));
                a_ring[s][h][e] = zero;
            }
    uint32_t e_ring[WIDE_STAGES][2 * MB];               // A8: the exponent bytes of those rows
    if constexpr (A8) {
#pragma unroll
        for (int s = 0; s < WIDE_STAGES; ++s)
#pragma unroll
            for (int h = 0; h < 2 * MB; ++h) {
                uint32_t zero;
                asm volatile("v_mov_b32 %0, 0" : "=v"(zero));
                e_ring[s][h] = zero;
            }
    }

    // Requests one unit: its 4 packed tiles straight into LDS stage S, its activations into a_ring[S] (inline assembly
    // for the loads and their waits, as in the 64-column kernel).
    auto fetch = [&](auto stage_tag) __attribute__((always_inline)) {
        constexpr int S = decltype(stage_tag)::value;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int l = 0; l < NLOAD; ++l)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(wptr[nb] + src_off[l]),
                                                 (__attribute__((address_space(3))) void *)(lds + wave * WAVE_LDS + S * UNIT_BYTES + nb * F::unit_bytes + l * F::load_stride),
                                                 16, 0, WEIGHTS_ONCE);
            wptr[nb] += w_step;
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            asm volatile("global_load_dwordx4 %0, %1, off" : "+v"(a_ring[S][2 * mb]) : "v"(aptr[mb]) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off" : "+v"(a_ring[S][2 * mb + 1]) : "v"(aptr[mb] + a_second) : "memory");
            aptr[mb] += a_step;
            if constexpr (A8) {
                asm volatile("global_load_ubyte %0, %1, off" : "+v"(e_ring[S][2 * mb]) : "v"(eptr[mb]) : "memory");
                asm volatile("global_load_ubyte %0, %1, off" : "+v"(e_ring[S][2 * mb + 1]) : "v"(eptr[mb] + 16) : "memory");
                eptr[mb] += a_step;
            }
        }
    };
    auto work = [&](auto stage_tag, auto younger_tag, bool refill) __attribute__((always_inline)) {
        constexpr int S = decltype(stage_tag)::value;
        constexpr int YOUNGER = decltype(younger_tag)::value;
        if (YOUNGER >= 0) wait_vmcnt<(YOUNGER < 0 ? 0 : YOUNGER) * PER>();   // < 0: the caller has waited
        if constexpr (MB == 2) asm volatile("" : "+v"(a_ring[S][0]), "+v"(a_ring[S][1]), "+v"(a_ring[S][2 * MB - 2]), "+v"(a_ring[S][2 * MB - 1]) :: "memory");
        else asm volatile("" : "+v"(a_ring[S][0]), "+v"(a_ring[S][1]) :: "memory");
        if constexpr (A8) {
#pragma unroll
            for (int s = 0; s < 2 * MB; ++s) asm volatile("" : "+v"(e_ring[S][s]) :: "memory");
        }
        u32x4 a_now[2 * MB];
#pragma unroll
        for (int s = 0; s < 2 * MB; ++s)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint32_t moved;
                asm volatile("v_mov_b32 %0, %1" : "=v"(moved) : "v"(a_ring[S][s][e]));
                a_now[s][e] = moved;
            }
        if constexpr (A8) {
            // codes and exponent -> 8 exact bf16 values, 64 times the activations (the factor leaves with the sums)
#pragma unroll
            for (int s = 0; s < 2 * MB; ++s) {
                uint32_t exponent;
                asm volatile("v_mov_b32 %0, %1" : "=v"(exponent) : "v"(e_ring[S][s]));
                a_now[s] = activations_operand8(kh ? a_now[s][2] : a_now[s][0], kh ? a_now[s][3] : a_now[s][1], exponent);
            }
        }
        // hidden-one form (bfp_dequant.h): A.W = 2 (A.hi - A.lo); the subtraction is an MFMA with the negated activations
        u32x4 a_neg[2 * MB];
#pragma unroll
        for (int s = 0; s < 2 * MB; ++s)
#pragma unroll
            for (int e = 0; e < 4; ++e) a_neg[s][e] = a_now[s][e] ^ 0x80008000u;
        // one weight matrix after the other; the stage is handed to the unit WIDE_STAGES ahead once its last LDS read has returned
        static_for(std::make_integer_sequence<int, NB>{}, [&](auto nb_tag) __attribute__((always_inline)) {
            constexpr int nb = decltype(nb_tag)::value;
            constexpr int AT = S * UNIT_BYTES + nb * F::unit_bytes;
            SlabRaw raw0, raw1;
            wide_slab_read<W, AT, AT>(exp_at, mant_at, raw0);
            wide_slab_read<W, AT + 32, AT + F::slab_bytes>(exp_at, mant_at, raw1);
            wait_slabs(raw0, raw1);
            if (nb == NB - 1 && refill) fetch(stage_tag);
            if constexpr (single_operand<W, MB>()) {
                bf16x8 bop[4];
                if constexpr (W == 3) slab_expand_bfp4(raw0, q, bop); else slab_expand_bfp8(raw0, bop);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[nb * MB + mb][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_now[2 * mb]), bop[j], acc[nb * MB + mb][j], 0, 0, 0);
                if constexpr (W == 3) slab_expand_bfp4(raw1, q, bop); else slab_expand_bfp8(raw1, bop);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[nb * MB + mb][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_now[2 * mb + 1]), bop[j], acc[nb * MB + mb][j], 0, 0, 0);
            } else {
                bf16x8 hi[4], lo[4];
                slab_expand_hidden<W>(raw0, q, hi, lo);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[nb * MB + mb][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_now[2 * mb]), hi[j], acc[nb * MB + mb][j], 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[nb * MB + mb][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_neg[2 * mb]), lo[j], acc[nb * MB + mb][j], 0, 0, 0);
                }
                slab_expand_hidden<W>(raw1, q, hi, lo);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[nb * MB + mb][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_now[2 * mb + 1]), hi[j], acc[nb * MB + mb][j], 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[nb * MB + mb][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_neg[2 * mb + 1]), lo[j], acc[nb * MB + mb][j], 0, 0, 0);
                }
            }
        });
    };

    // This wavefront's units: k_begin + wave, + WAVES, ...; unit i lives in stage i % STAGES and is requested STAGES
    // units ahead (see the 64-column kernel for the bookkeeping of requests in flight).
    const uint32_t span = k_end - k_begin;
    const bool computes = og < p.groups;             // the last `split` workgroups of a shared launch only collect
    const uint32_t total = computes && span > (uint32_t)wave ? (span - wave + WAVES - 1) / WAVES : 0;
    using Last = std::integral_constant<int, WIDE_STAGES - 1>;
    constexpr auto stages = std::make_integer_sequence<int, WIDE_STAGES>{};
    uint32_t i = 0;
    static_for(stages, [&](auto s) __attribute__((always_inline)) { if (total > (uint32_t)decltype(s)::value) fetch(s); });
    // steady state: every unit worked on here has a successor to request, so the number of requests in flight at each
    // wait is a constant the compiler can see
#pragma unroll 1
    for (; i + 2 * WIDE_STAGES <= total; i += WIDE_STAGES)
        static_for(stages, [&](auto s) __attribute__((always_inline)) { work(s, Last{}, true); });
    // at most 2 * STAGES - 1 units are left, starting in stage 0; the steps are nested (step J + 1 inside step J) so that
    // a step that does not happen takes all later ones with it
    nested_steps<0, 2 * WIDE_STAGES - 1>(i, total, [&](auto j) __attribute__((always_inline)) {
        constexpr int J = decltype(j)::value;
        const uint32_t at = i + J;
        wait_for_younger<WIDE_STAGES - 1, PER>(total - 1 - at);
        // a unit requested from here would be number J + STAGES of the tail: only the first STAGES - 1 steps can have one
        work(std::integral_constant<int, J % WIDE_STAGES>{}, std::integral_constant<int, -1>{}, J + WIDE_STAGES < 2 * WIDE_STAGES - 1 && at + WIDE_STAGES < total);
    });

    wait_vmcnt<0>();   // nothing in flight any more (already true; also what the build-time ISA check keys on)
    __builtin_amdgcn_sched_barrier(0);   // and nothing of what follows is scheduled in front of it
    // ---- add the four wavefronts' partial sums through LDS ------------------------------------------------------
    // One pass per set of sums (64 KB: the ring is empty by now): every wavefront writes its accumulator registers as float4
    // (acc[j][4q4 .. 4q4+3]); wavefront w then keeps q4 = w: rows 8w + 4kh + r (r = 0..3), columns 4*c32 + j.
    float4 *red = reinterpret_cast<float4 *>(lds);
    float mine[X][4][4];   // [set of sums][r][j]
#pragma unroll
    for (int nb = 0; nb < X; ++nb) {
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4)
                red[(wave * 16 + j * 4 + q4) * 64 + lane] = make_float4(acc[nb][j][4 * q4], acc[nb][j][4 * q4 + 1], acc[nb][j][4 * q4 + 2], acc[nb][j][4 * q4 + 3]);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int sw = 0; sw < WAVES; ++sw) {
                const float4 x = red[(sw * 16 + j * 4 + wave) * 64 + lane];
                v.x += x.x; v.y += x.y; v.z += x.z; v.w += x.w;
            }
            mine[nb][0][j] = v.x; mine[nb][1][j] = v.y; mine[nb][2][j] = v.z; mine[nb][3][j] = v.w;
        }
    }

    // ---- store, or hand over ------------------------------------------------------------------------------------
    // A chunk = 4 adjacent columns of one row = what one lane holds per r: chunk number (w * 4 + r) * 64 + lane, 1024
    // per output group.  Stores chunk `idx` of output group `group` (sums still carry the common factor; in the gated form
    // the activation applies to the first matrix's sums, which the second matrix's sums then multiply).
    // `mb` is the row band inside the group (two-band form).
    auto store_band = [&](uint32_t group, uint32_t idx, uint32_t mb, const float (&sums)[NB][4]) __attribute__((always_inline)) {
        const uint32_t lane_of = idx & 63, r_of = (idx >> 6) & 3, w_of = idx >> 8;
        const uint32_t c32_of = lane_of & 31, t_of = c32_of >> 3, fc_of = (c32_of >> 2) & 1, q_of = c32_of & 3;
        const uint32_t band_of = p.by_ngroups(group), bb_of = p.by_mt_sets(band_of), mt_of = (band_of - bb_of * p.mt_sets) * MB + mb;
        const uint32_t nt_of = (group - band_of * p.ngroups) * WIDE_TILES + t_of;
        const uint32_t row_in_band = w_of * 8 + (lane_of >> 5) * 4 + r_of, row = mt_of * 32 + row_in_band;
        if (nt_of >= p.nt || row >= p.m) return;
        const uint32_t n_col = nt_of * 32 + fc_of * 16 + q_of * 4;           // first of the 4 columns
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float x = sums[0][j] * (decode_unscale<W, MB>() * (A8 ? 0.015625f : 1.f));
            if (p.bias) x += __uint_as_float((uint32_t)p.bias[n_col + j] << 16);
            v[j] = apply_activation<ACT>(x);
            if (NB == 2) v[j] *= sums[NB - 1][j] * decode_unscale<W, MB>();
        }
        if (p.c_bfp) {
            // Block-float output (TILE layout): the sums are rounded to bf16 as for a bf16 output and packed with the host
            // packers' arithmetic; the shared exponent of the face row is a max over its 16 columns = this aligned lane quad.
            uint32_t bits[4], e_max = 0;
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                const uint32_t two = f32x2_to_bf16x2_rne(v[j], v[j + 1]);
                bits[j] = two << 16; bits[j + 1] = two & 0xffff0000u;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) e_max = max(e_max, (bits[j] >> 23) & 0xffu);
            const uint32_t shared = row_max<4>(e_max);
            const uint64_t tile = ((uint64_t)bb_of * p.mt + mt_of) * p.nt + nt_of;
            const uint32_t face = (row_in_band >> 4) * 2 + fc_of, row_in_face = row_in_band & 15;
            if (p.c_bfp == 7) {
                uint8_t *at = p.c + tile * 1088;
                const uint32_t word = to_code<7>(bits[0], shared) | (to_code<7>(bits[1], shared) << 8) | (to_code<7>(bits[2], shared) << 16) | (to_code<7>(bits[3], shared) << 24);
                *reinterpret_cast<uint32_t *>(at + 64 + face * 256 + row_in_face * 16 + q_of * 4) = word;
                if (q_of == 0) at[face * 16 + row_in_face] = (uint8_t)shared;
            } else {
                uint8_t *at = p.c + tile * 576;
                const uint32_t half = to_code<3>(bits[0], shared) | (to_code<3>(bits[1], shared) << 4) | (to_code<3>(bits[2], shared) << 8) | (to_code<3>(bits[3], shared) << 12);
                *reinterpret_cast<uint16_t *>(at + 64 + face * 128 + row_in_face * 8 + q_of * 2) = (uint16_t)half;
                if (q_of == 0) at[face * 16 + row_in_face] = (uint8_t)shared;
            }
            return;
        }
        uint64_t elem;   // element offset of the 4-column run in C
        if (p.c_tiled) {
            const uint64_t tile = ((uint64_t)bb_of * p.mt + mt_of) * p.nt + nt_of;
            elem = tile * 1024 + ((row_in_band >> 4) * 2 + fc_of) * 256 + (row_in_band & 15) * 16 + q_of * 4;
        } else {
            elem = ((uint64_t)bb_of * p.m + row) * p.n + n_col;
        }
        if (p.c_f32) {
            *reinterpret_cast<float4 *>(p.c + elem * 4) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
            const uint32_t lo16 = f32x2_to_bf16x2_rne(v[0], v[1]);
            const uint32_t hi16 = f32x2_to_bf16x2_rne(v[2], v[3]);
            *reinterpret_cast<uint2 *>(p.c + elem * 2) = make_uint2(lo16, hi16);
        }
    };

    // all sets of sums of a chunk: the two matrices of the gated form make one output, the two bands two
    auto store_chunk = [&](uint32_t group, uint32_t idx, const float (&sums)[X][4]) __attribute__((always_inline)) {
        if constexpr (MB == 1) {
            store_band(group, idx, 0, sums);
        } else {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                float one[NB][4];
#pragma unroll
                for (int j = 0; j < 4; ++j) one[0][j] = sums[mb][j];
                store_band(group, idx, mb, one);
            }
        }
    };

    if (p.split == 1) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float sums[X][4];
#pragma unroll
            for (int x = 0; x < X; ++x)
#pragma unroll
                for (int j = 0; j < 4; ++j) sums[x][j] = mine[x][r][j];
            store_chunk(og, (wave * 4 + r) * 64 + lane, sums);
        }
        return;
    }
    // Outputs shared between `split` workgroups.  Every workgroup publishes its 1024 chunks in its slot; the sums of
    // output group g are then formed by the `split` workgroups of the next group of the same XCD (g + 8; g + 1 where
    // placement is unknown; after the last group: by `split` workgroups launched for nothing else), workgroup j of them taking chunks [1024 j / split, 1024 (j + 1) / split)
    // from every contributor, in contributor order (so the result does not depend on timing), storing them and putting
    // SLOT_EMPTY back.  The work of collecting is spread evenly, every chunk is read by exactly one thread, and
    // whoever waits, waits for workgroups of lower index only: they were dispatched earlier and wait for nobody
    // dispatched later, so they finish.
    float4 *const all_slots = reinterpret_cast<float4 *>(p.slots);
    if (computes) {
        // slot (me, x) = 1024 chunks from chunk (me * X + x) * 1024 on
#pragma unroll
        for (int nb = 0; nb < X; ++nb) {
            float4 *slot = all_slots + (((uint64_t)me * X + nb) * 16 + wave * 4) * 64 + lane;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                u32x4 v;
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = not_empty(__float_as_uint(mine[nb][r][j]));
                if (p.drop_partial_sums) continue;
                if (in_xcds) slot_store_same_xcd(slot + r * 64, v); else slot_store(slot + r * 64, v);
            }
        }
    }
    if (og < before || og - before >= p.groups) return;
    const uint32_t target = og - before;
    // ranges of whole lane quads: the four chunks of a face row (16 columns) stay with four neighbouring threads
    const uint32_t lo = p.by_split(part * 256u) * 4u, hi = p.by_split((part + 1) * 256u) * 4u;
    const u32x4 empty = {SLOT_EMPTY, SLOT_EMPTY, SLOT_EMPTY, SLOT_EMPTY};
    for (uint32_t idx0 = lo; idx0 < hi; idx0 += 256) {
        const bool active = idx0 + threadIdx.x < hi;                       // idle lanes re-read the last chunk and drop it
        const uint32_t idx = active ? idx0 + threadIdx.x : hi - 1;
        float4 *const at = all_slots + (uint64_t)target * p.split * X * 1024 + idx;   // contributor c, set x: at + (c * X + x) * 1024
        uint32_t spins = 0;
        bool waiting;
        // workgroups with nothing else to do poll cheaply first (one contributor); then everything, checked word by word
        if (!computes) do {
            u32x4 probe = slot_load_issue(at + (uint64_t)(p.split * X - 1) * 1024);
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(probe)::"memory");
            const bool missing = active && (probe[0] == SLOT_EMPTY || probe[1] == SLOT_EMPTY || probe[2] == SLOT_EMPTY || probe[3] == SLOT_EMPTY);
            waiting = __ballot(missing) != 0 && ++spins < p.spin_limit;
            if (waiting) __builtin_amdgcn_s_sleep(8);
        } while (waiting);
        float sums[X][4];
#pragma unroll
        for (int x = 0; x < X; ++x)
#pragma unroll
            for (int j = 0; j < 4; ++j) sums[x][j] = 0.f;
        // N contributors at a time, N a compile-time constant: loads under a condition would have the compiler merge
        // loaded and unloaded registers (that is, copy them) while the loads are in flight
        auto collect = [&](auto count_tag, uint32_t c0) __attribute__((always_inline)) {
            constexpr int N = decltype(count_tag)::value * X;           // slots: those of a contributor lie side by side
            u32x4 got[N];
            do {
#pragma unroll
                for (int u = 0; u < N; ++u) got[u] = slot_load_issue(at + ((uint64_t)c0 * X + u) * 1024);
#pragma unroll
                for (int u = 0; u < N; ++u) asm volatile("s_waitcnt vmcnt(0)" : "+v"(got[u])::"memory");
                bool missing = false;
#pragma unroll
                for (int u = 0; u < N; ++u)
#pragma unroll
                    for (int j = 0; j < 4; ++j) missing |= got[u][j] == SLOT_EMPTY;
                const bool any_missing = __ballot(missing && active) != 0;
                waiting = any_missing && ++spins < p.spin_limit;
                if (waiting) __builtin_amdgcn_s_sleep(4);
                else if (any_missing) report_timeout(p);
            } while (waiting);
#pragma unroll
            for (int u = 0; u < N; ++u) {
#pragma unroll
                for (int j = 0; j < 4; ++j) sums[u % X][j] += __uint_as_float(got[u][j]);
                if (active) { if (in_xcds) slot_store_same_xcd(at + ((uint64_t)c0 * X + u) * 1024, empty); else slot_store(at + ((uint64_t)c0 * X + u) * 1024, empty); }       // ready for the next launch
            }
        };
        uint32_t c0 = 0;
        for (; c0 + 8 <= p.split; c0 += 8) collect(std::integral_constant<int, 8>{}, c0);
        switch (p.split - c0) {
            case 1: collect(std::integral_constant<int, 1>{}, c0); break;
            case 2: collect(std::integral_constant<int, 2>{}, c0); break;
            case 3: collect(std::integral_constant<int, 3>{}, c0); break;
            case 4: collect(std::integral_constant<int, 4>{}, c0); break;
            case 5: collect(std::integral_constant<int, 5>{}, c0); break;
            case 6: collect(std::integral_constant<int, 6>{}, c0); break;
            case 7: collect(std::integral_constant<int, 7>{}, c0); break;
            default: break;
        }
        if (active) store_chunk(target, idx, sums);
    }
}

// ---------------------------------------------------------------------------------------------------------
// host side: decomposition, workspace, launch
// ---------------------------------------------------------------------------------------------------------
struct Decomposition { uint32_t mt, mt_sets, kt, nt, ngroups, workgroups, split; uint64_t groups, units; };

// two_bands: the 128-column kernel takes two 32-row bands per workgroup (33 to 127 rows, not gated)
static bool two_bands(uint32_t m, bool wide, bool gated) { return wide && !gated && m > 32; }

// 64-column kernel: between 200 and 256 output groups are one workgroup per CU, each with its whole k range: nothing is
// handed over (with fewer groups too many CUs idle, with more a second round begins).
static bool one_round_of_groups(uint64_t groups) { return groups >= 200 && groups <= 256; }

static Decomposition decompose(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, bool wide, bool gated = false) {
    Decomposition d{};
    const uint32_t group_tiles = wide ? WIDE_TILES : GROUP_TILES;
    d.mt = (m + 31) / 32; d.kt = k / 32; d.nt = n / 32;
    d.mt_sets = two_bands(m, wide, gated) ? (d.mt + 1) / 2 : d.mt;
    d.ngroups = (d.nt + group_tiles - 1) / group_tiles;
    d.groups = (uint64_t)batch * d.mt_sets * d.ngroups;
    d.units = d.groups * d.kt;
    // Workgroups to aim for, every output's k range being cut into as many parts as get there (every wavefront keeping
    // >= 2 k-tiles).  64-column kernel: 256 CUs x 3 workgroups of 4 wavefronts when the output groups alone nearly get
    // there, x 2 otherwise (every extra k range of an output costs a slot store, a slot read and a slot reset).  128-column kernel: two
    // workgroups per CU (all it can hold, the collecting workgroups included) when that takes few parts per output, one
    // per CU when the outputs are few (measured: many short k ranges cost more than the second workgroup gains).
    // The gated form does twice the work per workgroup and hands over twice as much: one workgroup per CU, i.e. half as
    // many k ranges per output (measured on Mistral's gate / up shape: 25.3-25.8 us against 26.3 us with two per CU).
    const bool few = d.groups < 100 || gated;
    const uint64_t resident = knob_or(TTMI_KNOB_MATMUL_WORKGROUPS, wide ? (few ? 256 : 256 * WIDE_WGS_PER_CU) : d.groups >= 256 ? 768 : 512);
    uint64_t parts = d.groups >= resident ? 1 : wide && !few ? resident / (d.groups + 1) : resident / d.groups;
    // The round of workgroups that only collect may come late (they are the last of the launch and wait for everybody
    // anyway): where counting them in leaves a quarter of the places empty and one more k range per output fills them
    // exactly, take it, if every wavefront still keeps 8 k-tiles.  Measured: [32, 4544] x [4544, 16384] (128 groups)
    // 20.8-21.3 us with 4 ranges against 23.6-24.0 with 3; [4544, 21760] (170 groups) 25.8-26.1 with 3 against 30.9-31.6
    // with 2; [8192, 16384] 30.7-31.5 against 36.3-36.9.  (More ranges than that cost more than they fill:
    // [4544, 13056], 102 groups, 22.2-22.9 us with 5 against 19.2-19.7 with 4.)
    if (wide && !few && d.groups < resident && d.groups * parts * 100 < resident * 78 && d.groups * (parts + 1) <= resident && d.kt >= 8u * WAVES * (parts + 1))
        ++parts;
    uint32_t asked;
    if (!wide && one_round_of_groups(d.groups) && !knob(TTMI_KNOB_MATMUL_WORKGROUPS, &asked)) parts = 1;
    if (parts == 0) parts = 1;
    const uint64_t most = d.kt / (2 * WAVES) ? d.kt / (2 * WAVES) : 1;
    if (parts > most) parts = most;
    d.split = (uint32_t)parts;
    d.workgroups = (uint32_t)(d.groups * parts);
    return d;
}

static size_t slot_bytes_needed(const Decomposition &d, bool wide, bool two_sets = false) {
    if (d.split == 1) return 0;                     // every output belongs to one workgroup: no slot is touched
    return wide ? (size_t)d.workgroups * WIDE_SLOT_BYTES * (two_sets ? 2 : 1) : (size_t)2 * d.workgroups * SLOT_BYTES;
}

// Where consecutive workgroups run.  The 128-column kernel keeps the workgroups that share an output in one XCD, which
// relies on consecutive workgroups going to consecutive XCDs, eight of them: workgroup b to XCD (b + c) % 8 with some c
// that is the same for the whole launch (observed on MI355X from the null stream, from other streams, back to back,
// beside a kernel on another stream and in graph replays; c depends on the queue).  A probe launch reads the XCC_ID
// register of 64 workgroups once per device; any other answer — another part, a partitioned one — selects the
// device-scope hand-over, which assumes nothing about placement.
static __device__ uint32_t placement_probe[64];
__global__ void placement_probe_kernel(uint32_t *out) {
    uint32_t xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    if (threadIdx.x == 0) out[blockIdx.x] = xcc & 0xfu;
}
static std::mutex g_placement_guard;
static uint32_t g_xcds[64];       // per device, 0 = not asked yet

static int device_xcds(uint32_t *xcds) {
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (dev < 0 || dev >= 64) return fail(TTMI_ERR_UNSUPPORTED, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_placement_guard);
    if (!g_xcds[dev]) {
        uint32_t *probe = nullptr;
        if (int rc = check_hip(hipGetSymbolAddress((void **)&probe, HIP_SYMBOL(placement_probe)), "hipGetSymbolAddress(placement_probe)")) return rc;
        hipLaunchKernelGGL(placement_probe_kernel, dim3(64), dim3(64), 0, nullptr, probe);
        if (int rc = check_launch("placement_probe_kernel")) return rc;
        uint32_t seen[64];
        if (int rc = check_hip(hipMemcpy(seen, probe, sizeof(seen), hipMemcpyDeviceToHost), "hipMemcpy(placement_probe)")) return rc;
        bool round_robin = true;
        for (uint32_t b = 0; b < 64; ++b) round_robin = round_robin && seen[b] == (seen[0] + b) % 8;
        g_xcds[dev] = round_robin ? 8 : 1;
    }
    *xcds = g_xcds[dev];
    return TTMI_OK;
}

// Dealing the output groups out to 8 XCDs leaves some XCDs a group short when their number is no multiple of 8: only where
// that costs little (at most 1/32 of a round).
static bool deal_to_xcds(const Decomposition &d) { return d.split > 1 && (((uint32_t)d.groups + 7) / 8) * 8 * 32 <= (uint32_t)d.groups * 33; }
static uint32_t wide_grid_size(const Decomposition &d, bool in_xcds) {
    return d.split == 1 ? d.workgroups : in_xcds ? 8 * (((uint32_t)d.groups + 7) / 8 + 1) * d.split : d.workgroups + d.split;
}

static int launch_streaming(const MatmulArgs &x, hipStream_t st, bool wide) {
    const Decomposition d = decompose(x.batch, x.m, x.k, x.n, wide, x.b2 != nullptr);
    MatmulDev p{};
    p.a = (const uint8_t *)x.a; p.b = (const uint8_t *)x.b; p.b2 = (const uint8_t *)x.b2; p.bias = (const uint16_t *)x.bias; p.c = (uint8_t *)x.c;
    const bool gated = x.b2 != nullptr;
    if (gated && !wide) return fail(TTMI_ERR_UNSUPPORTED, "matmul: the gated form runs on the 128-column kernel only");
    const bool a8 = x.a_dtype == TTMI_BFLOAT8_B;
    if (a8 && !(wide && !gated && x.m <= 32 && x.a_layout == TTMI_TILE)) return fail(TTMI_ERR_UNSUPPORTED, "matmul: this kernel takes no block-float activations");
    p.batch = x.batch; p.b_batch = x.b_batch; p.m = x.m; p.k = x.k; p.n = x.n;
    p.mt = d.mt; p.mt_sets = d.mt_sets; p.kt = d.kt; p.nt = d.nt; p.ngroups = d.ngroups; p.groups = (uint32_t)d.groups; p.workgroups = d.workgroups; p.units = (uint32_t)d.units;
    p.split = d.split;
    p.by_split = fast_div(d.split); p.by_ngroups = fast_div(d.ngroups); p.by_mt_sets = fast_div(d.mt_sets);
    p.a_tiled = x.a_layout == TTMI_TILE; p.c_tiled = x.c_layout == TTMI_TILE;
    p.c_f32 = x.c_dtype == TTMI_FLOAT32;
    p.c_bfp = x.c_dtype == TTMI_BFLOAT8_B ? 7 : x.c_dtype == TTMI_BFLOAT4_B ? 3 : 0;
    if (p.c_bfp && !(wide && p.c_tiled)) return fail(TTMI_ERR_UNSUPPORTED, "matmul: this kernel writes no block-float output");
    if ((reinterpret_cast<uintptr_t>(x.a) | reinterpret_cast<uintptr_t>(x.b) | reinterpret_cast<uintptr_t>(x.b2) | reinterpret_cast<uintptr_t>(x.c)) & 15u)
        return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: a, b and c must be 16-byte aligned");
    if (d.units > 0x7fffffffull || d.groups * d.split > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: problem too large for one launch");
    const bool bands2 = two_bands(x.m, wide, gated);
    const size_t need = slot_bytes_needed(d, wide, gated || bands2);
    void *slots = nullptr;
    bool fill = false;
    size_t fill_bytes = need;
    if (need == 0) {
    } else if (x.workspace) {
        if (x.workspace_bytes < need) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: workspace of %zu bytes given, %zu needed", x.workspace_bytes, need);
        if (reinterpret_cast<uintptr_t>(x.workspace) & 255u) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: workspace must be 256-byte aligned");
        slots = x.workspace;
        fill = need > x.workspace_empty_bytes;      // a caller's buffer may hold anything, unless it says how much of it is empty slots
        if (x.workspace_left_empty_bytes) *x.workspace_left_empty_bytes = std::max(need, x.workspace_empty_bytes);      // a launch that completes leaves its slots empty
    } else if (int rc = scratch_get(SCRATCH_SLOTS, st, need, &slots, &fill, &fill_bytes)) {
        // the library's own slots, one buffer per stream: every word is SLOT_EMPTY once filled, and every launch that
        // completes leaves it that way
        return rc;
    }
    if (fill) {
        // every slot becomes empty: of a caller's workspace those of this launch, of the library's buffer all it can hold
        // (a later launch that needs more of them is not told that the buffer is fresh); with a kernel, not a memset
        // node: the caller may be capturing the stream into a graph
        const uint32_t chunks = (uint32_t)(fill_bytes / 16);
        hipLaunchKernelGGL(fill_slots_kernel, dim3((chunks + 255) / 256 < 2048 ? (chunks + 255) / 256 : 2048), dim3(256), 0, st, (u32x4 *)slots, chunks);
        if (int rc = check_launch("fill_slots_kernel")) return rc;
    }
    p.slots = (float *)slots;
    if (x.no_alloc) {
        // a report lands in the device's error word when one exists (any earlier ttmi_device_status() creates it),
        // otherwise in the last bytes of the workspace, where nobody looks: the wait is bounded either way
        if (!error_word_if_exists(&p.error, nullptr))
            p.error = x.workspace ? reinterpret_cast<uint32_t *>((uint8_t *)x.workspace + x.workspace_bytes - 256) : nullptr;   // no workspace: nothing is shared, nobody waits
    } else if (int rc = error_word(&p.error, nullptr)) {
        return rc;
    }
    p.spin_limit = knob_or(TTMI_KNOB_SPIN_LIMIT, SLOT_SPIN_LIMIT);
    p.drop_partial_sums = (int)knob_or(TTMI_KNOB_DROP_PARTIAL_SUMS, 0);      // always 0 in the product library
    // 128-column kernel with shared outputs: one more round of `split` workgroups per XCD collects the XCD's last groups
    p.xcds = 1;
    if (wide && d.split > 1 && p.error)
        if (int rc = device_xcds(&p.xcds)) return rc;
    if (p.xcds == 8 && !deal_to_xcds(d)) p.xcds = 1;
    p.xcds = knob_or(TTMI_KNOB_XCDS, p.xcds) == 8 ? p.xcds : 1;      // a test can ask for the placement-agnostic form
    const uint32_t wide_grid = wide_grid_size(d, p.xcds == 8);
#define TTMI_LAUNCH(W, ACT)                                                                                     \
    if (wide && gated) hipLaunchKernelGGL((matmul_wide_kernel<W, ACT, 2, 1>), dim3(wide_grid), dim3(256), 0, st, p); \
    else if (wide && a8) hipLaunchKernelGGL((matmul_wide_kernel<W, ACT, 1, 1, true>), dim3(wide_grid), dim3(256), 0, st, p); \
    else if (wide && bands2) hipLaunchKernelGGL((matmul_wide_kernel<W, ACT, 1, 2>), dim3(wide_grid), dim3(256), 0, st, p); \
    else if (wide) hipLaunchKernelGGL((matmul_wide_kernel<W, ACT, 1, 1>), dim3(wide_grid), dim3(256), 0, st, p); \
    else hipLaunchKernelGGL((matmul_stream_kernel<W, ACT>), dim3(d.workgroups), dim3(256), 0, st, p)
#define TTMI_LAUNCH_ACT(W)                                              \
    switch (x.activation) {                                             \
        case TTMI_ACT_RELU: TTMI_LAUNCH(W, TTMI_ACT_RELU); break;       \
        case TTMI_ACT_GELU: TTMI_LAUNCH(W, TTMI_ACT_GELU); break;       \
        case TTMI_ACT_SILU: TTMI_LAUNCH(W, TTMI_ACT_SILU); break;       \
        default: TTMI_LAUNCH(W, TTMI_ACT_NONE); break;                  \
    }
    if (x.b_fmt == TTMI_BFLOAT8_B) { TTMI_LAUNCH_ACT(7) } else { TTMI_LAUNCH_ACT(3) }
#undef TTMI_LAUNCH_ACT
#undef TTMI_LAUNCH
    return check_launch(wide ? "matmul_wide_kernel" : "matmul_stream_kernel");
}

int matmul_bfp_stream(const MatmulArgs &x, hipStream_t st) { return launch_streaming(x, st, false); }
int matmul_bfp_wide(const MatmulArgs &x, hipStream_t st) { return launch_streaming(x, st, true); }

// Which kernel a shape goes to.  Up to 127 rows the weights are streamed (HBM-bound): one 32-row band in 128-column units;
// two or four bands in the two-band form of the same kernel, which streams the weights once per 64 rows (measured at 64
// rows, TILE layout: 32.8 against 44.1 us for the Falcon h_to_4h shape, 29.8 against 41.4 us for 4h_to_h, no difference for
// Mistral's shapes); three bands in 64-column units, once per band, when the GEMM has more columns than rows of weights,
// else in the two-band form, whose fourth band is computed for nothing but which cuts a long k range finer (measured at 96
// rows, 64-column against two-band: [4544, 18176] BFP8_B 56.5 against 73.2 us, [4096, 14336] BFP4_B 32.0 against 33.7; but
// [18176, 4544] BFP8_B 58.1 against 54.0, [4096, 4096] BFP8_B 17.6 against 15.6, [14336, 4096] BFP4_B 37.0 against 30.3).  Taller activations are MFMA-bound: the fused tiled kernels up to 511 rows, and from 512 rows
// on (two or more 256-row blocks share every weight) the weights are expanded to bf16 once and a plain bf16 GEMM follows.
// The test entry point can force a kernel (TTMI_KNOB_MATMUL_KERNEL).
enum class Kernel { Stream = 1, Wide = 2, Tile = 3, Expanded = 4 };
static Kernel choose_kernel(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt, bool c_bfp) {
    uint32_t forced;
    if (knob(TTMI_KNOB_MATMUL_KERNEL, &forced) && forced >= 1 && forced <= 4) return (Kernel)forced;
    if (m >= 128) {
        // Tall activations are MFMA-bound when the output has enough blocks for the chip: a 128 x 256 or 256 x 256 block per
        // workgroup takes about 0.75 us per k-tile, and a GEMM with few columns leaves most CUs without one.  Streaming the
        // weights once per 64 rows (the two-band form of the 128-column kernel, which cuts the k range to fill the chip)
        // is then faster, up to surprisingly many rows.  Measured, BFLOAT8_B, one MI355X: [256, 4096] x [4096, 4096] 28 us
        // against 102 (tiled) and 85 (expanded); [128, 14336] x [14336, 4096] 34 against 331 and 264; [256, 4096] x
        // [4096, 14336] 54 against 103 and 105; [448, 4544] x [4544, 18176] 138 against 229 and 130; 12 x [384, 1024] x
        // [1024, 1024] 29.5 against 24.8 (the 384-row kernel).  The estimates below reproduce those within 15 %.
        const double k_tiles = k / 32, weights = (double)k * n * (b_fmt == TTMI_BFLOAT8_B ? 1.0625 : 0.8);     // BFLOAT4_B: half the bytes, the same instructions
        const double sets = (double)batch * (((m + 31) / 32 + 1) / 2);
        const double streamed_us = 8.0 + sets * weights / 4.7e6;
        double blocked_us;
        if (m >= 512) {
            const double blocks = (double)batch * ((m + 255) / 256) * ((n + 255) / 256);
            blocked_us = 4.0 + (double)k * n * 3.0625 / 6.0e6 + std::ceil(blocks / 256.0) * k_tiles * 0.72;      // expansion pass + bf16 GEMM
        } else {
            const double blocks = (double)batch * ((m + 127) / 128) * ((n + 255) / 256);
            blocked_us = std::ceil(blocks / 256.0) * k_tiles * 0.78;
        }
        if (streamed_us < 0.9 * blocked_us) return Kernel::Wide;
        return m >= 512 ? Kernel::Expanded : Kernel::Tile;
    }
    // One band of BFP4_B weights whose 64-column groups are one workgroup per CU, with at most 192 KiB of weights each:
    // the 64-column kernel, which then shares no output and has nothing to hand over.  Measured against the 128-column
    // kernel, same box, M = 32, weights rotated through more than the Infinity Cache holds: [4096, 14336] BFP4_B (Mistral's
    // gate / up, 147 KB per group) 15.0 against 15.3 us, [4096, 16384] BFP4_B 15.2 against 18.7, [2048, 15360] BFP4_B 9.7
    // against 10.8; but [8192, 14336] BFP4_B (295 KB) 25.3 against 23.0, and BFP8_B loses at every size ([2048, 14336]
    // 12.3 against 11.7, [4096, 12800] 18.0 against 17.7, [8192, 14336] 30.0 against 28.4): the longer the k range, the
    // less the hand-over matters and the more the 64-column kernel's extra instruction work per byte.  It writes no
    // block-float output.
    const uint64_t group_weights = (uint64_t)(k / 32) * GROUP_TILES * 576u;
    if (m <= 32 && !c_bfp && b_fmt == TTMI_BFLOAT4_B && group_weights <= 192u * 1024u &&
        one_round_of_groups((uint64_t)batch * ((n / 32 + GROUP_TILES - 1) / GROUP_TILES)))
        return Kernel::Stream;
    return m <= 32 || ((m + 31) / 32) % 2 == 0 || c_bfp || k >= n ? Kernel::Wide : Kernel::Stream;
}

size_t matmul_gated_workspace_bytes(uint32_t batch, uint32_t m, uint32_t k, uint32_t n) {
    if (!batch || !m || !k || !n) return 0;
    return slot_bytes_needed(decompose(batch, m, k, n, true, true), true, true);
}

size_t matmul_workspace_bytes(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt) {
    if (!batch || !m || !k || !n) return 0;
    const Kernel kernel = choose_kernel(batch, m, k, n, b_fmt, false);
    switch (kernel) {
        case Kernel::Expanded: return matmul_expanded_workspace_bytes(batch, k, n);   // as if every slice had weights of its own
        case Kernel::Tile: return 0;
        default: break;
    }
    const bool wide = kernel == Kernel::Wide;
    const size_t need = slot_bytes_needed(decompose(batch, m, k, n, wide), wide, two_bands(m, wide, false));
    // 64-column kernel: with a block-float output the same shape goes to the 128-column kernel
    if (!wide) return std::max(need, slot_bytes_needed(decompose(batch, m, k, n, true), true, two_bands(m, true, false)));
    return need;
}

// What a shape gets: the kernel, the k ranges per output and the grid (for reading profiler output; no GPU needed).
void matmul_plan(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt, bool a_or_c_bfp, uint32_t out[4]) {
    out[0] = out[1] = out[2] = out[3] = 0;
    if (!batch || !m || !k || !n) return;
    const Kernel kernel = choose_kernel(batch, m, k, n, b_fmt, a_or_c_bfp);
    out[0] = (uint32_t)kernel;
    if (kernel != Kernel::Wide && kernel != Kernel::Stream) return;
    const bool wide = kernel == Kernel::Wide;
    const Decomposition d = decompose(batch, m, k, n, wide);
    out[1] = d.split;
    out[2] = wide ? wide_grid_size(d, false) : d.workgroups;
    out[3] = wide && deal_to_xcds(d) ? wide_grid_size(d, true) : out[2];
}

bool matmul_takes_bfp_activations(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt) {
    // One band of rows: with two, the expansion of four slabs of activations per unit no longer fits the registers beside
    // two sets of sums (measured with it: [64, 18176] x [18176, 4544] 45.5 us against 38.3 for expanding A first).
    return batch && m == 32 && k && n && choose_kernel(batch, m, k, n, b_fmt, true) == Kernel::Wide;
}

int matmul_bfp(const MatmulArgs &x, hipStream_t st) {
    // what an earlier launch on this device has reported (a wait for partial sums that gave up) surfaces here
    if (!x.no_alloc || error_word_if_exists(nullptr, nullptr))
        if (int rc = ttmi_device_status()) return rc;
    // every kernel but the 64-column one packs a block-float output in its epilogue (choose_kernel keeps that one out of it)
    const bool c_bfp = x.c_dtype == TTMI_BFLOAT8_B || x.c_dtype == TTMI_BFLOAT4_B;
    const bool a8 = x.a_dtype == TTMI_BFLOAT8_B;      // block-float activations: the 128-column kernel alone takes them
    const Kernel kernel = choose_kernel(x.batch, x.m, x.k, x.n, x.b_fmt, c_bfp || a8);
    if (a8 && !matmul_takes_bfp_activations(x.batch, x.m, x.k, x.n, x.b_fmt))
        return fail(TTMI_ERR_UNSUPPORTED, "matmul: block-float activations are taken by the one-band streaming kernel only, which this shape does "
                    "not go to (ttmi_matmul_bfp_ab_supported): expand them with ttmi_typecast_tiles first");
    switch (kernel) {
        case Kernel::Expanded: return matmul_bfp_expanded(x, st);
        case Kernel::Tile: return matmul_bfp_tiled(x, st);
        case Kernel::Wide: return matmul_bfp_wide(x, st);
        default: return matmul_bfp_stream(x, st);
    }
}

// bf16 x bf16: the weights are brought into the operand layout of the expanding GEMM's second pass (a re-layout instead of
// an expansion), whatever the number of rows.
int matmul_bf16(const MatmulArgs &x, hipStream_t st) {
    if (int rc = ttmi_device_status()) return rc;
    return matmul_bfp_expanded(x, st);
}

// c = act(a . b + bias) * (a . b2) in one launch of the 128-column kernel (any number of rows: the weights are streamed
// once per 32-row band, so it is meant for decode shapes).
int matmul_bfp_gated(const MatmulArgs &x, hipStream_t st) {
    if (int rc = ttmi_device_status()) return rc;
    return launch_streaming(x, st, true);
}

}  // namespace ttmi

// ---------------------------------------------------------------------------------------------------------
// ttmi_matmul_bfp for callers that cannot allocate (a stream under graph capture, a serving loop that forbids hipMalloc):
// the scratch of the kernels — partial-sum slots below 128 rows, expanded weights from 512 rows on — lies in a static
// device array instead of a buffer that the library allocates on first use.  Every GPU that the library runs on holds its
// own copy of the array, at its own address, until the process ends; all calls on one GPU share it.
// ---------------------------------------------------------------------------------------------------------
static __device__ __align__(256) uint8_t scratch[TTMI_STATIC_SCRATCH_BYTES + 256];      // + 256: stand-in for the error word
static void *g_scratch_at[64];       // device address of `scratch` per device (the array's name is no device address on the host)
// How many leading bytes of the array hold nothing but empty partial-sum slots, per device (a launch that shares outputs
// then needs no fill launch in front of it), as of which generation of the library's slot buffers (a reported give-up
// invalidates them all).  Kernels that put expanded weights into the array set it back to 0.
static size_t g_scratch_empty_bytes[64];
static uint64_t g_scratch_generation[64];
static std::mutex g_scratch_guard;

static int static_scratch(void **ptr) {
    int dev = 0;
    if (int rc = ttmi::check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (dev < 0 || dev >= 64) return ttmi::fail(TTMI_ERR_UNSUPPORTED, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_guard);
    if (!g_scratch_at[dev]) {
        void *at = nullptr;
        if (int rc = ttmi::check_hip(hipGetSymbolAddress(&at, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return rc;
        g_scratch_at[dev] = at;
    }
    *ptr = g_scratch_at[dev];
    return TTMI_OK;
}

extern "C" int ttmi_matmul_bfp_static(const void *a, int a_layout, const uint32_t *b, int b_fmt, uint32_t batch, uint32_t b_batch,
                                      uint32_t m, uint32_t k, uint32_t n, const void *bias, int activation, void *c, int c_layout,
                                      int c_dtype, void *stream) {
    if (int rc = ttmi::validate_matmul(a, a_layout, b, b_fmt, batch, b_batch, m, k, n, activation, c, c_layout, c_dtype)) return rc;
    const size_t need = ttmi::matmul_workspace_bytes(batch, m, k, n, b_fmt);
    if (need > TTMI_STATIC_SCRATCH_BYTES)
        return ttmi::fail(TTMI_ERR_UNSUPPORTED, "matmul (static scratch): this shape needs %zu bytes of scratch, the static array holds %zu; "
                          "use ttmi_matmul_bfp with a workspace", need, (size_t)TTMI_STATIC_SCRATCH_BYTES);
    void *at = nullptr;
    if (need)
        if (int rc = static_scratch(&at)) return rc;
    ttmi::MatmulArgs args{a, a_layout, b, b_fmt, batch, b_batch, m, k, n, bias, activation, c, c_layout, c_dtype, at, need ? (size_t)TTMI_STATIC_SCRATCH_BYTES + 256 : 0};
    args.no_alloc = true;
    int dev = 0;
    if (int rc = ttmi::check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    size_t left_empty = 0;
    {
        std::lock_guard<std::mutex> lock(g_scratch_guard);
        const uint64_t generation = ttmi::scratch_generation(ttmi::SCRATCH_SLOTS);
        args.workspace_empty_bytes = g_scratch_generation[dev] == generation ? g_scratch_empty_bytes[dev] : 0;
        g_scratch_generation[dev] = generation;
        g_scratch_empty_bytes[dev] = 0;     // until this call has gone through: it may put expanded weights there instead
    }
    args.workspace_left_empty_bytes = &left_empty;
    const int rc = ttmi::matmul_bfp(args, (hipStream_t)stream);
    if (rc == TTMI_OK && left_empty) {
        std::lock_guard<std::mutex> lock(g_scratch_guard);
        g_scratch_empty_bytes[dev] = left_empty;
    }
    return rc;
}

#ifdef TTMI_TEST_HOOKS
// Test entry points (not declared in include/ttmi.h): the decomposition the host chooses for a shape, and the two index
// functions the kernels cut the work with, so that their invariants can be checked without a GPU.
// Test entry point: the LDS stage of the 128-column kernel as its code computes it, for lane `lane` of a wavefront.
//   out[0] loads per unit, out[1] bytes between the LDS destinations of consecutive loads, out[2] stage bytes,
//   out[3] bytes from slab 0 to slab 1 (mantissas), out[4] bytes between the two rows of a ds_read2_b32,
//   out[5..8] byte offsets of the four ds_read2_b32 of a slab, out[9] exponent address, out[10] mantissa address
//   (both inside the stage, slab 0), out[11..] the chunk of the unit that the lane fetches in every load
template <int W> static void wide_layout_of(int lane, uint32_t *out) {
    using F = ttmi::WideFmt<W>;
    const int c32 = lane & 31, kh = lane >> 5, t = c32 >> 3, fc = (c32 >> 2) & 1, q = c32 & 3;
    out[0] = F::loads; out[1] = F::load_stride; out[2] = F::unit_bytes; out[3] = F::slab_bytes; out[4] = F::row_step;
    for (int i = 0; i < 4; ++i) out[5 + i] = F::pair_offset(i);
    out[9] = ttmi::wide_exp_at<W>(t, fc, kh); out[10] = ttmi::wide_mant_at<W>(t, fc, q, kh);
    uint32_t chunk_of[F::loads];
    ttmi::wide_stage_chunks<W>(lane, chunk_of);
    for (int l = 0; l < F::loads; ++l) out[11 + l] = chunk_of[l];
}
extern "C" {
__attribute__((visibility("default"))) void ttmi_test_stream_decomposition(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int wide,
                                                                           uint32_t out[4]) {
    const ttmi::Decomposition d = ttmi::decompose(batch, m, k, n, wide != 0);
    out[0] = (uint32_t)d.groups; out[1] = d.kt; out[2] = d.split; out[3] = d.workgroups;
}
// which kernel a shape goes to: 1 = 64-column streaming kernel, 2 = 128-column streaming kernel, 3 = tiled, 4 = expanded
__attribute__((visibility("default"))) int ttmi_test_kernel_choice(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt, int c_dtype) {
    return (int)ttmi::choose_kernel(batch, m, k, n, b_fmt, c_dtype == TTMI_BFLOAT8_B || c_dtype == TTMI_BFLOAT4_B);
}
__attribute__((visibility("default"))) void ttmi_test_wide_layout(int mantissa_bits, int lane, uint32_t out[16]) {
    if (mantissa_bits == 7) wide_layout_of<7>(lane, out); else wide_layout_of<3>(lane, out);
}
__attribute__((visibility("default"))) uint32_t ttmi_test_range_start(uint32_t kt, uint32_t split, uint32_t i) { return ttmi::range_start(kt, split, i); }
// 128-column kernel, output groups dealt out to 8 XCDs: group * split + part of the workgroup with hardware index b
__attribute__((visibility("default"))) uint32_t ttmi_test_wide_workgroup_number(uint32_t b, uint32_t split) { return ttmi::wide_workgroup_number(b, split, ttmi::fast_div(split)); }
// n / d as the kernels compute it
__attribute__((visibility("default"))) uint32_t ttmi_test_fast_div(uint32_t n, uint32_t d) { return ttmi::fast_div(d)(n); }
__attribute__((visibility("default"))) uint32_t ttmi_test_workgroup_of(uint32_t kt, uint32_t split, uint32_t unit) { return ttmi::workgroup_of(kt, split, unit); }
}
#endif
