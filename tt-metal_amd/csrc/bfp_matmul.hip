// GEMM with block-float weights for gfx950:  C[b,m,n] = act(A[b,m,k] . W[(b|0),k,n] + bias[n]).
//
// Semantics follow tt::operations::primary::matmul (tt_eager/tt_dnn/op_library/bmm/bmm_op.hpp:318-346,
// bmm_op.cpp:828-1049): bf16 activations, BFLOAT8_B / BFLOAT4_B weights stored as packed 32x32 tiles
// (tile (kt, nt) at index kt*Nt + nt; layout of one tile: tt_metal/common/bfloat8.hpp:102-173), fp32
// accumulation, bf16 (or fp32) output.  Weight values are what the reference unpacker produces
// (bfloat8.hpp:229-249, tt_metal/common/bfloat4.hpp:113-146): sign * mantissa * 2^(E - 127 - (W-1)); they
// carry at most 7 significant bits, so the conversion to bf16 in front of the matrix cores is exact.
//
// streaming kernel (one 32-row band of A per workgroup; decode shapes)
//   workgroup = 4 wavefronts = one (32-row m band, 128-column n group, k range); the wavefronts take the
//   k-tiles of the range round-robin, so every packed weight byte is read from HBM exactly once per m band.
//   Per k-tile a wavefront copies 4 adjacent packed tiles (one contiguous run) into its private LDS slice,
//   then for each 16-row half issues four v_mfma_f32_32x32x16_bf16: lane (c, g) holds, for MFMA j,
//   column 4c+j of the group and k rows 8g..8g+7 — byte j of the 8 mantissa words it read — so no transposed
//   copy of the weights is ever made.  Partial sums of the 4 wavefronts meet in LDS; each wavefront then owns
//   8 rows x 128 columns of the result and stores them as contiguous runs.
//   With more than one k range per output the fp32 partials go to a workspace and a second kernel sums them.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "ttmi_internal.h"

namespace ttmi {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

struct MatmulDev {
    const uint8_t *a;        // bf16
    const uint8_t *b;        // packed tiles
    const uint16_t *bias;    // bf16 [n] or null
    uint8_t *c;              // output (bf16 or fp32)
    float *partial;          // [ksplit][batch*m][n] when ksplit > 1
    uint32_t batch, b_batch, m, k, n;
    uint32_t mt, kt, nt, ngroups, ksplit, kt_per_split;
    int a_tiled, c_tiled, c_f32, activation;
};

template <int W> struct Wfmt;
template <> struct Wfmt<7> {
    static constexpr int tile_bytes = 1088, chunks = 68, rows_per_chunk = 1, row_bytes = 16;
    static constexpr int face_stride = 320, tile_stride = 1296;     // LDS strides of the mantissa area (padded)
    static constexpr int bias_exp = 133;
};
template <> struct Wfmt<3> {
    static constexpr int tile_bytes = 576, chunks = 36, rows_per_chunk = 2, row_bytes = 8;
    static constexpr int face_stride = 144, tile_stride = 608;
    static constexpr int bias_exp = 129;
};

constexpr int GROUP_TILES = 4;                       // n tiles per workgroup
constexpr int WAVES = 4;
constexpr int EXP_AREA = GROUP_TILES * 64;           // exponent bytes of the 4 staged tiles
constexpr int REDUCE_BYTES = WAVES * 48 * 64 * 4;    // 48 fp32 per lane handed over per wavefront

template <int W> constexpr int stage_bytes() { return EXP_AREA + GROUP_TILES * Wfmt<W>::tile_stride; }

__device__ __forceinline__ float apply_activation(float x, int act) {
    switch (act) {
        case TTMI_ACT_RELU: return x > 0.f ? x : 0.f;
        case TTMI_ACT_GELU: return 0.5f * x * (1.f + erff(x * 0.70710678118654752440f));
        case TTMI_ACT_SILU: return x / (1.f + __expf(-x));
        default: return x;
    }
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float x) {
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// Eight weights of one output column, k rows 8g..8g+7, as the bf16 B operand of one MFMA.
//   words[jj]  mantissa word of k row 8g+jj that contains this column's code
//   scale[jj]  2^(E - bias_exp) of that row
//   sel        which code inside the word (byte 0..3 for W=7, nibble 0..7 for W=3)
template <int W>
__device__ __forceinline__ bf16x8 weights_operand(const uint32_t (&words)[8], const float (&scale)[8], int sel) {
    uint32_t packed[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        uint32_t half[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const uint32_t code = words[2 * p + s] >> ((W + 1) * sel);
            const float mag = (float)(code & ((1u << W) - 1u)) * scale[2 * p + s];
            half[s] = (__float_as_uint(mag) >> 16) | (((code >> W) & 1u) << 15);
        }
        packed[p] = half[0] | (half[1] << 16);
    }
    return __builtin_bit_cast(bf16x8, make_uint4(packed[0], packed[1], packed[2], packed[3]));
}

template <int W>
__global__ __launch_bounds__(256) void matmul_stream_kernel(const MatmulDev p) {
    using F = Wfmt<W>;
    constexpr int STAGE = stage_bytes<W>();
    constexpr int LDS_BYTES = REDUCE_BYTES > WAVES * STAGE ? REDUCE_BYTES : WAVES * STAGE;
    constexpr int NLOAD = (GROUP_TILES * F::chunks + 63) / 64;
    __shared__ __attribute__((aligned(16))) uint8_t lds[LDS_BYTES];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 31, g = lane >> 5;
    const int t_of_lane = c >> 3, fc = (c >> 2) & 1, q = c & 3;

    uint32_t idx = blockIdx.x;
    const uint32_t ks = idx % p.ksplit; idx /= p.ksplit;
    const uint32_t ng = idx % p.ngroups; idx /= p.ngroups;
    const uint32_t mt = idx % p.mt;
    const uint32_t bb = idx / p.mt;
    const uint32_t nt0 = ng * GROUP_TILES;
    const uint32_t n_valid = min((uint32_t)GROUP_TILES, p.nt - nt0);
    const uint32_t kt_begin = ks * p.kt_per_split;
    const uint32_t kt_end = min(p.kt, kt_begin + p.kt_per_split);

    const uint8_t *wbase = p.b + (uint64_t)(p.b_batch == 1 ? 0 : bb) * p.kt * p.nt * F::tile_bytes;
    uint8_t *my_stage = lds + wave * STAGE;
    uint8_t *my_mant = my_stage + EXP_AREA;

    f32x16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;

    const uint32_t chunks_valid = n_valid * F::chunks;
    uint4 inflight[NLOAD];
    auto fetch = [&](uint32_t kt) {
        const uint4 *src = reinterpret_cast<const uint4 *>(wbase + ((uint64_t)kt * p.nt + nt0) * F::tile_bytes);
#pragma unroll
        for (int l = 0; l < NLOAD; ++l) {
            const uint32_t gch = l * 64 + lane;
            inflight[l] = gch < chunks_valid ? src[gch] : make_uint4(0, 0, 0, 0);
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int l = 0; l < NLOAD; ++l) {
            const uint32_t gch = l * 64 + lane;
            if (gch >= GROUP_TILES * F::chunks) continue;
            const uint32_t t = gch / F::chunks, r = gch % F::chunks;
            uint8_t *to;
            if (r < 4) to = my_stage + t * 64 + r * 16;
            else {
                const uint32_t rr = r - 4;                       // 16-byte chunk inside the mantissa area
                const uint32_t per_face = 16 / F::rows_per_chunk;
                to = my_mant + t * F::tile_stride + (rr / per_face) * F::face_stride + (rr % per_face) * 16;
            }
            *reinterpret_cast<uint4 *>(to) = inflight[l];
        }
    };

    const uint32_t m_row = mt * 32 + c;       // activation row this lane feeds to the MFMA
    uint32_t kt = kt_begin + wave;
    if (kt < kt_end) fetch(kt);
    for (; kt < kt_end; kt += WAVES) {
        stash();
        if (kt + WAVES < kt_end) fetch(kt + WAVES);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            // activations: rows m, k = kt*32 + h*16 + g*8 .. +7
            uint4 araw = make_uint4(0, 0, 0, 0);
            if (p.a_tiled) {
                const uint8_t *at = p.a + (((uint64_t)bb * p.mt + mt) * p.kt + kt) * 2048 + ((c >> 4) * 2 + h) * 512 +
                                    (c & 15) * 32 + g * 16;
                araw = *reinterpret_cast<const uint4 *>(at);
            } else if (m_row < p.m) {
                const uint8_t *at = p.a + (((uint64_t)bb * p.m + m_row) * p.k + kt * 32 + h * 16 + g * 8) * 2;
                araw = *reinterpret_cast<const uint4 *>(at);
            }
            const bf16x8 aop = __builtin_bit_cast(bf16x8, araw);

            const int face = 2 * h + fc;
            const uint2 e2 = *reinterpret_cast<const uint2 *>(my_stage + t_of_lane * 64 + face * 16 + g * 8);
            float scale[8];
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) {
                const uint32_t e = ((jj < 4 ? e2.x : e2.y) >> (8 * (jj & 3))) & 0xffu;
                scale[jj] = ldexpf(1.0f, (int)e - F::bias_exp);
            }
            uint32_t words[8];
            const uint8_t *rows = my_mant + t_of_lane * F::tile_stride + face * F::face_stride + (g * 8) * F::row_bytes;
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) {
                if (W == 7) words[jj] = *reinterpret_cast<const uint32_t *>(rows + jj * 16 + q * 4);
                else words[jj] = *reinterpret_cast<const uint32_t *>(rows + jj * 8 + (q >> 1) * 4) >> (16 * (q & 1));
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bf16x8 bop = weights_operand<W>(words, scale, j);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aop, bop, acc[j], 0, 0, 0);
            }
        }
    }

    // hand over: wavefront w keeps accumulator registers 4w..4w+3 of all four MFMAs (rows 8w + 4g + 0..3)
    __syncthreads();
    float *red = reinterpret_cast<float *>(lds);
#pragma unroll
    for (int ow = 0; ow < WAVES; ++ow) {
        if (ow == wave) continue;
        const int slot = ow < wave ? ow : ow - 1;     // 3 slots per source wavefront
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                red[(((wave * 3 + slot) * 16) + j * 4 + r) * 64 + lane] = acc[j][ow * 4 + r];
    }
    __syncthreads();
    float mine[4][4];   // [r][j]
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) mine[r][j] = acc[j][wave * 4 + r];
#pragma unroll
    for (int sw = 0; sw < WAVES; ++sw) {
        if (sw == wave) continue;
        const int slot = wave < sw ? wave : wave - 1;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) mine[r][j] += red[(((sw * 3 + slot) * 16) + j * 4 + r) * 64 + lane];
    }

    if (t_of_lane >= (int)n_valid) return;
    const uint32_t n_col = (nt0 + t_of_lane) * 32 + fc * 16 + q * 4;   // first of this lane's 4 columns
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t row_in_band = wave * 8 + g * 4 + r;
        const uint32_t row = mt * 32 + row_in_band;
        if (row >= p.m) continue;
        if (p.ksplit > 1) {
            float *to = p.partial + ((uint64_t)ks * p.batch * p.m + (uint64_t)bb * p.m + row) * p.n + n_col;
            *reinterpret_cast<float4 *>(to) = make_float4(mine[r][0], mine[r][1], mine[r][2], mine[r][3]);
            continue;
        }
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float x = mine[r][j];
            if (p.bias) x += __uint_as_float((uint32_t)p.bias[n_col + j] << 16);
            v[j] = apply_activation(x, p.activation);
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
            const uint32_t lo = f32_to_bf16_rne(v[0]) | ((uint32_t)f32_to_bf16_rne(v[1]) << 16);
            const uint32_t hi = f32_to_bf16_rne(v[2]) | ((uint32_t)f32_to_bf16_rne(v[3]) << 16);
            *reinterpret_cast<uint2 *>(p.c + elem * 2) = make_uint2(lo, hi);
        }
    }
}

// Sums the k-range partials, applies bias / activation, converts and stores in the output layout.
__global__ __launch_bounds__(256) void matmul_finish_kernel(const MatmulDev p) {
    const uint64_t quads = (uint64_t)p.batch * p.m * (p.n / 4);
    const uint64_t at = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= quads) return;
    const uint32_t n_col = (uint32_t)(at % (p.n / 4)) * 4;
    const uint64_t brow = at / (p.n / 4);        // b*m + row
    const uint32_t row = (uint32_t)(brow % p.m);
    const uint32_t bb = (uint32_t)(brow / p.m);
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    for (uint32_t ks = 0; ks < p.ksplit; ++ks) {
        const float4 v = *reinterpret_cast<const float4 *>(p.partial + ((uint64_t)ks * p.batch * p.m + brow) * p.n + n_col);
        sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
    }
    float v[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (p.bias) v[j] += __uint_as_float((uint32_t)p.bias[n_col + j] << 16);
        v[j] = apply_activation(v[j], p.activation);
    }
    uint64_t elem;
    if (p.c_tiled) {
        const uint32_t mt = row >> 5, rin = row & 31, nt = n_col >> 5, cin = n_col & 31;
        const uint64_t tile = ((uint64_t)bb * p.mt + mt) * p.nt + nt;
        elem = tile * 1024 + ((rin >> 4) * 2 + (cin >> 4)) * 256 + (rin & 15) * 16 + (cin & 15);
    } else {
        elem = brow * p.n + n_col;
    }
    if (p.c_f32) {
        *reinterpret_cast<float4 *>(p.c + elem * 4) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
        const uint32_t lo = f32_to_bf16_rne(v[0]) | ((uint32_t)f32_to_bf16_rne(v[1]) << 16);
        const uint32_t hi = f32_to_bf16_rne(v[2]) | ((uint32_t)f32_to_bf16_rne(v[3]) << 16);
        *reinterpret_cast<uint2 *>(p.c + elem * 2) = make_uint2(lo, hi);
    }
}

// ---------------------------------------------------------------------------------------------------------
// host side: split selection, workspace, launch
// ---------------------------------------------------------------------------------------------------------
static uint32_t env_u32(const char *name, uint32_t fallback) {
    const char *v = getenv(name);
    if (!v || !*v) return fallback;
    const long x = strtol(v, nullptr, 10);
    return x > 0 ? (uint32_t)x : fallback;
}

static uint32_t choose_ksplit(uint32_t batch, uint32_t m, uint32_t k, uint32_t n) {
    const uint32_t mt = (m + 31) / 32, kt = k / 32, nt = n / 32;
    const uint32_t base = batch * mt * ((nt + GROUP_TILES - 1) / GROUP_TILES);
    const uint32_t forced = env_u32("TTMI_MATMUL_KSPLIT", 0);
    uint32_t split = forced ? forced : (env_u32("TTMI_MATMUL_TARGET_WGS", 768) + base - 1) / base;
    const uint32_t max_split = kt / WAVES ? kt / WAVES : 1;   // every wavefront gets at least one k-tile
    if (split > max_split) split = max_split;
    if (split < 1) split = 1;
    const uint32_t per = (kt + split - 1) / split;
    return (kt + per - 1) / per;                              // drop empty ranges
}

size_t matmul_workspace_bytes(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int) {
    if (!batch || !m || !k || !n) return 0;
    const uint32_t split = choose_ksplit(batch, m, k, n);
    return split > 1 ? (size_t)split * batch * m * n * sizeof(float) : 0;
}

// The library's own scratch, one per device, grown on demand and kept until the process ends.
static void *g_scratch[64] = {nullptr};
static size_t g_scratch_bytes[64] = {0};

static int own_scratch(size_t bytes, void **out) {
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (dev < 0 || dev >= 64) return fail(TTMI_ERR_UNSUPPORTED, "device index %d out of range", dev);
    if (g_scratch_bytes[dev] < bytes) {
        if (g_scratch[dev]) {
            if (int rc = check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize")) return rc;
            if (int rc = check_hip(hipFree(g_scratch[dev]), "hipFree")) return rc;
            g_scratch[dev] = nullptr; g_scratch_bytes[dev] = 0;
        }
        if (int rc = check_hip(hipMalloc(&g_scratch[dev], bytes), "hipMalloc(matmul scratch)")) return rc;
        g_scratch_bytes[dev] = bytes;
    }
    *out = g_scratch[dev];
    return TTMI_OK;
}

int matmul_bfp(const MatmulArgs &x, hipStream_t st) {
    MatmulDev p{};
    p.a = (const uint8_t *)x.a; p.b = (const uint8_t *)x.b; p.bias = (const uint16_t *)x.bias; p.c = (uint8_t *)x.c;
    p.batch = x.batch; p.b_batch = x.b_batch; p.m = x.m; p.k = x.k; p.n = x.n;
    p.mt = (x.m + 31) / 32; p.kt = x.k / 32; p.nt = x.n / 32;
    p.ngroups = (p.nt + GROUP_TILES - 1) / GROUP_TILES;
    p.ksplit = choose_ksplit(x.batch, x.m, x.k, x.n);
    p.kt_per_split = (p.kt + p.ksplit - 1) / p.ksplit;
    p.a_tiled = x.a_layout == TTMI_TILE; p.c_tiled = x.c_layout == TTMI_TILE;
    p.c_f32 = x.c_dtype == TTMI_FLOAT32; p.activation = x.activation;
    if ((reinterpret_cast<uintptr_t>(x.a) | reinterpret_cast<uintptr_t>(x.b) | reinterpret_cast<uintptr_t>(x.c)) & 15u)
        return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: a, b and c must be 16-byte aligned");
    const uint64_t blocks = (uint64_t)p.batch * p.mt * p.ngroups * p.ksplit;
    if (blocks > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: problem too large for one launch");
    if (p.ksplit > 1) {
        const size_t need = (size_t)p.ksplit * p.batch * p.m * p.n * sizeof(float);
        void *ws = x.workspace;
        if (ws) {
            if (x.workspace_bytes < need) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: workspace of %zu bytes given, %zu needed", x.workspace_bytes, need);
            if (reinterpret_cast<uintptr_t>(ws) & 15u) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: workspace must be 16-byte aligned");
        } else if (int rc = own_scratch(need, &ws)) {
            return rc;
        }
        p.partial = (float *)ws;
    }
    if (x.b_fmt == TTMI_BFLOAT8_B) hipLaunchKernelGGL(matmul_stream_kernel<7>, dim3((uint32_t)blocks), dim3(256), 0, st, p);
    else hipLaunchKernelGGL(matmul_stream_kernel<3>, dim3((uint32_t)blocks), dim3(256), 0, st, p);
    if (int rc = check_launch("matmul_stream_kernel")) return rc;
    if (p.ksplit > 1) {
        const uint64_t quads = (uint64_t)p.batch * p.m * (p.n / 4);
        hipLaunchKernelGGL(matmul_finish_kernel, dim3((uint32_t)((quads + 255) / 256)), dim3(256), 0, st, p);
        if (int rc = check_launch("matmul_finish_kernel")) return rc;
    }
    return TTMI_OK;
}

}  // namespace ttmi
