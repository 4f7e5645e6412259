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
//              registers), two units ahead of the arithmetic; per unit it builds four B operands and issues eight
//              v_mfma_f32_16x16x32_bf16.  Lane (c, g) — c = lane % 16, g = lane / 16 — holds, for operand j, column
//              4c+j of the group and k rows 8g..8g+7: byte j of the 8 mantissa words it reads from LDS.  The packed
//              layout (16 consecutive columns of one k row share a word run) never has to be transposed.
//   workgroup  4 wavefronts take the units of a contiguous range round-robin, add their partial sums through LDS
//              and store; the range is this workgroup's equal share of ALL units ("stream-K"), so every workgroup
//              streams the same number of bytes whatever K and N are.  Outputs whose k range is shared between
//              workgroups are finished by the workgroup that arrives last (see the kernel).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <type_traits>

#include "bfp_dequant.h"
#include "ttmi_internal.h"

namespace ttmi {

struct MatmulDev {
    const uint8_t *a;        // bf16
    const uint8_t *b;        // packed tiles
    const uint16_t *bias;    // bf16 [n] or null
    uint8_t *c;              // output (bf16 or fp32)
    float *slots;            // 2 slots of 32x64 fp32 per workgroup, for outputs shared between workgroups
    uint32_t *counters;      // one arrival counter per output group (all zero between launches)
    uint32_t batch, b_batch, m, k, n;
    uint32_t mt, kt, nt, ngroups;
    uint32_t workgroups;     // P
    uint32_t units;          // U = batch * mt * ngroups * kt
    uint32_t share, extra;   // U = P * share + extra: the first `extra` workgroups take share + 1 units
    uint32_t split;          // k ranges per output group, or 0 for stream-K
    int a_tiled, c_tiled, c_f32;
};

constexpr int GROUP_TILES = 2;                       // n tiles per output group
constexpr int GROUP_COLS = GROUP_TILES * 32;
constexpr int WAVES = 4;
constexpr int STAGES = 3;                            // LDS ring per wavefront: two units in flight, one in use
constexpr int REDUCE_BYTES = WAVES * 32 * 64 * 4;    // every wavefront lays out its 32 accumulator registers
constexpr size_t SLOT_BYTES = 32 * GROUP_COLS * sizeof(float);

// Partial sums that other workgroups read travel through device-coherent accesses: relaxed atomic stores and loads
// at agent scope go past the per-XCD L2 (which is not coherent across XCDs), so no cache write-back or invalidate
// is needed — a full agent-scope fence here costs more than the whole GEMM.
__device__ __forceinline__ void slot_store(float4 *to, const float4 v) {
    uint64_t *q = reinterpret_cast<uint64_t *>(to);
    __hip_atomic_store(q, ((uint64_t)__float_as_uint(v.y) << 32) | __float_as_uint(v.x), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(q + 1, ((uint64_t)__float_as_uint(v.w) << 32) | __float_as_uint(v.z), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float4 slot_load(const float4 *from) {
    uint64_t *q = reinterpret_cast<uint64_t *>(const_cast<float4 *>(from));
    const uint64_t lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_float4(__uint_as_float((uint32_t)lo), __uint_as_float((uint32_t)(lo >> 32)), __uint_as_float((uint32_t)hi),
                       __uint_as_float((uint32_t)(hi >> 32)));
}

// Which units a workgroup takes.
//   split > 0   every output group is cut into `split` nearly equal k ranges, one per workgroup (P = groups * split):
//               one output per workgroup, at most `split` partial sums to add
//   split == 0  "stream-K": the U units are dealt out contiguously, the first `extra` workgroups take share + 1 units,
//               the rest `share`; a range may end one output and begin the next
__device__ __forceinline__ uint32_t range_start(const MatmulDev &p, uint32_t i) {
    if (p.split) return (i / p.split) * p.kt + ((i % p.split) * p.kt) / p.split;
    return i * p.share + min(i, p.extra);
}
__device__ __forceinline__ uint32_t workgroup_of(const MatmulDev &p, uint32_t unit) {
    if (p.split) {
        const uint32_t og = unit / p.kt, within = unit - og * p.kt;
        return og * p.split + ((within + 1) * p.split - 1) / p.kt;     // largest part j with (j * kt) / split <= within
    }
    const uint32_t fat = p.extra * (p.share + 1);
    return unit < fat ? unit / (p.share + 1) : p.extra + (unit - fat) / p.share;
}

// Work decomposition ("stream-K"): units are numbered with the k-tile fastest and dealt out contiguously and
// evenly to P workgroups (P = what the chip holds at once).  A workgroup whose range covers all k-tiles of an
// output group stores that output directly.  Otherwise it writes its fp32 partial sums to a slot of its own and
// bumps the group's arrival counter; the workgroup that arrives last adds the slots in workgroup order (so the
// result does not depend on who was last), applies the epilogue, stores, and resets the counter.
template <int W, int ACT>
__global__ __launch_bounds__(256, 3) void matmul_stream_kernel(const MatmulDev p) {
    using F = Wfmt<W>;
    constexpr int WAVE_LDS = STAGES * F::stage_bytes;
    constexpr int LDS_BYTES = REDUCE_BYTES > WAVES * WAVE_LDS ? REDUCE_BYTES : WAVES * WAVE_LDS;
    constexpr int NLOAD = F::loads;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[LDS_BYTES];
    __shared__ uint32_t arrival;

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
    u32x4 a_next[2];                                  // activations of the unit after the one being worked on
    uint32_t src_off[NLOAD];
    uint32_t a_half = 0;                              // bytes from row c to row c + 16 of the band (set per segment)
    const uint8_t *wptr = nullptr, *aptr = nullptr;

    // Requests the 2 packed tiles of one unit straight into LDS stage `stage` (wavefront-uniform).
    auto fetch_weights = [&](uint32_t stage) {
#pragma unroll
        for (int l = 0; l < NLOAD; ++l)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(wptr + src_off[l]),
                                             (__attribute__((address_space(3))) void *)(lds + wave * WAVE_LDS + stage * F::stage_bytes + l * 1024),
                                             16, 0, 0);
        wptr += w_step;
    };
    auto fetch_activations = [&]() {
        a_next[0] = *reinterpret_cast<const u32x4 *>(aptr);
        a_next[1] = *reinterpret_cast<const u32x4 *>(aptr + a_half);
        aptr += a_step;
    };
    // Works on the unit in the stage at `stage_off` with activations (a_lo, a_hi).
    auto compute = [&](uint32_t stage_off, const bf16x8 a_lo, const bf16x8 a_hi, auto after_lds_reads) {
        bf16x8 bop[4];
        staged_operands<W>(lds, stage_off + exp_off, stage_off + mant_off, q, after_lds_reads, bop);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, bop[j], acc[0][j], 0, 0, 0);
            acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, bop[j], acc[1][j], 0, 0, 0);
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

        // This wavefront's units: k_begin + wave, + WAVES, ... (`total` of them).  Unit i lives in stage i % STAGES.
        // Vector-memory operations complete in order, so they are issued in this order:
        //   weights(0), weights(1), activations(0) | per unit i: activations(i+1), [LDS reads of i], weights(i+2), math
        // At the top of unit i everything but the youngest weights request must have landed: vmcnt(NLOAD) while a
        // request is still young, vmcnt(0) at the tail.
        const uint32_t span = k_end - k_begin;
        const uint32_t total = span > (uint32_t)wave ? (span - wave + WAVES - 1) / WAVES : 0;
        if (total > 0) fetch_weights(0);
        if (total > 1) fetch_weights(1);
        if (total > 0) fetch_activations();
        uint32_t stage = 0;
#pragma unroll 1
        for (uint32_t i = 0; i < total; ++i) {
            if (i >= 1 && i + 1 < total) wait_vmcnt<NLOAD>(); else if (i == 0 && total > 1) wait_vmcnt<NLOAD>(); else wait_vmcnt<0>();
            const bf16x8 a_lo = __builtin_bit_cast(bf16x8, a_next[0]), a_hi = __builtin_bit_cast(bf16x8, a_next[1]);
            if (i + 1 < total) fetch_activations();
            const uint32_t refill_stage = stage == 0 ? STAGES - 1 : stage - 1;     // (i + 2) % STAGES
            compute(stage * F::stage_bytes, a_lo, a_hi, [&]() { if (i + 2 < total) fetch_weights(refill_stage); });
            stage = stage + 1 == STAGES ? 0 : stage + 1;
        }

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
        bool store_now = true;
        if (k_begin != 0 || k_end != p.kt) {
            // contributors: workgroups first..last, the ones whose ranges meet [og*kt, (og+1)*kt)
            const uint32_t lo = og * p.kt;
            const uint32_t first = workgroup_of(p, lo), last = workgroup_of(p, lo + p.kt - 1);
            float4 *slot = reinterpret_cast<float4 *>(p.slots) + ((uint64_t)(2 * me + (og == my_first_og ? 0 : 1)) * 8 + wave * 2) * 64 + lane;
#pragma unroll
            for (int r = 0; r < 2; ++r) slot_store(slot + r * 64, make_float4(mine[r][0], mine[r][1], mine[r][2], mine[r][3]));
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");   // our slot stores have completed ...
            __syncthreads();
            if (threadIdx.x == 0)                                    // ... before the arrival is announced
                arrival = __hip_atomic_fetch_add(&p.counters[og], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            store_now = arrival == last - first;
            if (store_now) {
                float sum[2][4];
#pragma unroll
                for (int r = 0; r < 2; ++r)
#pragma unroll
                    for (int j = 0; j < 4; ++j) sum[r][j] = 0.f;
                // fixed order (the result does not depend on who is last), four contributors' loads in flight at a time
                for (uint32_t w0 = first; w0 <= last; w0 += 4) {
                    float4 part[4][2];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const uint32_t w = min(w0 + u, last);
                        const uint32_t which = range_start(p, w) >= lo ? 0u : 1u;      // first or second output of w
                        const float4 *other = reinterpret_cast<const float4 *>(p.slots) + ((uint64_t)(2 * w + which) * 8 + wave * 2) * 64 + lane;
#pragma unroll
                        for (int r = 0; r < 2; ++r) part[u][r] = slot_load(other + r * 64);
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const uint32_t w = w0 + u;
                        if (w > last) break;
#pragma unroll
                        for (int r = 0; r < 2; ++r) {
                            const float4 v = w == me ? make_float4(mine[r][0], mine[r][1], mine[r][2], mine[r][3]) : part[u][r];
                            sum[r][0] += v.x; sum[r][1] += v.y; sum[r][2] += v.z; sum[r][3] += v.w;
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < 2; ++r)
#pragma unroll
                    for (int j = 0; j < 4; ++j) mine[r][j] = sum[r][j];
                if (threadIdx.x == 0) __hip_atomic_store(&p.counters[og], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
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
                    float x = mine[r][j];
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
                    const uint32_t lo16 = f32_to_bf16_rne(v[0]) | ((uint32_t)f32_to_bf16_rne(v[1]) << 16);
                    const uint32_t hi16 = f32_to_bf16_rne(v[2]) | ((uint32_t)f32_to_bf16_rne(v[3]) << 16);
                    *reinterpret_cast<uint2 *>(p.c + elem * 2) = make_uint2(lo16, hi16);
                }
            }
        }
        __syncthreads();   // LDS is reused by the next segment
    }
}

// ---------------------------------------------------------------------------------------------------------
// host side: decomposition, workspace, launch
// ---------------------------------------------------------------------------------------------------------
static uint32_t env_u32(const char *name, uint32_t fallback) {
    const char *v = getenv(name);
    if (!v || !*v) return fallback;
    const long x = strtol(v, nullptr, 10);
    return x > 0 ? (uint32_t)x : fallback;
}

struct Decomposition { uint32_t mt, kt, nt, ngroups, workgroups, split; uint64_t groups, units; };

static Decomposition decompose(uint32_t batch, uint32_t m, uint32_t k, uint32_t n) {
    Decomposition d{};
    d.mt = (m + 31) / 32; d.kt = k / 32; d.nt = n / 32;
    d.ngroups = (d.nt + GROUP_TILES - 1) / GROUP_TILES;
    d.groups = (uint64_t)batch * d.mt * d.ngroups;
    d.units = d.groups * d.kt;
    // workgroups in flight at once: 256 CUs x 3 workgroups of 4 wavefronts measured best (4 fit)
    const uint64_t resident = env_u32("TTMI_MATMUL_WGS", 768);
    if (env_u32("TTMI_MATMUL_STREAMK", 0)) {
        d.split = 0;
        d.workgroups = (uint32_t)(d.units < resident ? d.units : resident);
    } else {
        // cut every output's k range into as many parts as keeps the chip full, every wavefront keeping >= 2 k-tiles
        uint64_t parts = d.groups >= resident ? 1 : resident / d.groups;
        const uint64_t most = d.kt / (2 * WAVES) ? d.kt / (2 * WAVES) : 1;
        if (parts > most) parts = most;
        d.split = (uint32_t)parts;
        d.workgroups = (uint32_t)(d.groups * parts);
    }
    return d;
}

static size_t counters_bytes(const Decomposition &d) { return (d.groups * sizeof(uint32_t) + 255) / 256 * 256; }

size_t matmul_workspace_bytes(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int) {
    if (!batch || !m || !k || !n) return 0;
    const Decomposition d = decompose(batch, m, k, n);
    return counters_bytes(d) + (size_t)2 * d.workgroups * SLOT_BYTES;
}

// The library's own scratch, per device, grown on demand and kept until the process ends: arrival counters
// (zeroed when allocated; every launch leaves them at zero again) and partial-sum slots.  They are separate
// allocations so that slot data of one problem size can never be read as counters of another.
struct Scratch { void *ptr = nullptr; size_t bytes = 0; };
static Scratch g_counters[64], g_slots[64];

static int grow(Scratch &s, size_t bytes, bool zero) {
    if (s.bytes >= bytes) return TTMI_OK;
    if (s.ptr) {
        if (int rc = check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize")) return rc;
        if (int rc = check_hip(hipFree(s.ptr), "hipFree")) return rc;
        s.ptr = nullptr; s.bytes = 0;
    }
    if (int rc = check_hip(hipMalloc(&s.ptr, bytes), "hipMalloc(matmul scratch)")) return rc;
    if (zero) if (int rc = check_hip(hipMemset(s.ptr, 0, bytes), "hipMemset(matmul scratch)")) return rc;
    s.bytes = bytes;
    return TTMI_OK;
}

static int own_scratch(size_t counter_bytes, size_t slot_bytes, void **counters, void **slots) {
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (dev < 0 || dev >= 64) return fail(TTMI_ERR_UNSUPPORTED, "device index %d out of range", dev);
    if (int rc = grow(g_counters[dev], counter_bytes, true)) return rc;
    if (int rc = grow(g_slots[dev], slot_bytes, false)) return rc;
    *counters = g_counters[dev].ptr;
    *slots = g_slots[dev].ptr;
    return TTMI_OK;
}

int matmul_bfp_stream(const MatmulArgs &x, hipStream_t st) {
    const Decomposition d = decompose(x.batch, x.m, x.k, x.n);
    MatmulDev p{};
    p.a = (const uint8_t *)x.a; p.b = (const uint8_t *)x.b; p.bias = (const uint16_t *)x.bias; p.c = (uint8_t *)x.c;
    p.batch = x.batch; p.b_batch = x.b_batch; p.m = x.m; p.k = x.k; p.n = x.n;
    p.mt = d.mt; p.kt = d.kt; p.nt = d.nt; p.ngroups = d.ngroups; p.workgroups = d.workgroups; p.units = (uint32_t)d.units;
    p.share = p.units / p.workgroups; p.extra = p.units % p.workgroups; p.split = d.split;
    p.a_tiled = x.a_layout == TTMI_TILE; p.c_tiled = x.c_layout == TTMI_TILE;
    p.c_f32 = x.c_dtype == TTMI_FLOAT32;
    if ((reinterpret_cast<uintptr_t>(x.a) | reinterpret_cast<uintptr_t>(x.b) | reinterpret_cast<uintptr_t>(x.c)) & 15u)
        return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: a, b and c must be 16-byte aligned");
    if (d.units > 0x7fffffffull || d.groups * (d.split ? d.split : 1) > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: problem too large for one launch");
    const size_t slot_bytes = (size_t)2 * d.workgroups * SLOT_BYTES, need = counters_bytes(d) + slot_bytes;
    void *counters = nullptr, *slots = nullptr;
    if (x.workspace) {
        if (x.workspace_bytes < need) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: workspace of %zu bytes given, %zu needed", x.workspace_bytes, need);
        if (reinterpret_cast<uintptr_t>(x.workspace) & 255u) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: workspace must be 256-byte aligned");
        // a caller's buffer may hold anything: clear the arrival counters for this launch
        if (int rc = check_hip(hipMemsetAsync(x.workspace, 0, counters_bytes(d), st), "hipMemsetAsync(counters)")) return rc;
        counters = x.workspace;
        slots = (uint8_t *)x.workspace + counters_bytes(d);
    } else if (int rc = own_scratch(counters_bytes(d), slot_bytes, &counters, &slots)) {
        return rc;
    }
    p.counters = (uint32_t *)counters;
    p.slots = (float *)slots;
#define TTMI_LAUNCH(W, ACT) hipLaunchKernelGGL((matmul_stream_kernel<W, ACT>), dim3(d.workgroups), dim3(256), 0, st, p)
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
    return check_launch("matmul_stream_kernel");
}

// Tall activations are MFMA-bound and go to the tiled kernel; up to 127 rows the weights are streamed once per
// 32-row band.  TTMI_MATMUL_KERNEL=stream|tile overrides the choice (for tests and measurements).
int matmul_bfp(const MatmulArgs &x, hipStream_t st) {
    const char *force = getenv("TTMI_MATMUL_KERNEL");
    if (force && force[0] == 's') return matmul_bfp_stream(x, st);
    if (force && force[0] == 't') return matmul_bfp_tiled(x, st);
    return x.m >= 128 ? matmul_bfp_tiled(x, st) : matmul_bfp_stream(x, st);
}

}  // namespace ttmi
