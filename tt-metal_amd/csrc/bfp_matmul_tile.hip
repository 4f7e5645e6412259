// Tiled GEMM with block-float weights for gfx950, for tall activations (prefill, batched bmm): MFMA-bound.
//
//   workgroup  4 wavefronts compute a (16*MB)-row x 256-column block of C (MB = 16 or 8); the k loop advances one
//              packed tile (32 rows of W) at a time through a ring of LDS stages filled by direct global->LDS loads
//   A          the block's rows x 32 k values of bf16 go to LDS as they lie in memory (64 bytes per row) and are
//              shared by the 4 wavefronts; a 16-row A operand of v_mfma_f32_16x16x32_bf16 is one ds_read_b128 per lane
//   W          every wavefront owns 64 columns = 2 packed tiles per k step, staged in the layout of Wfmt and expanded
//              straight into B operands (byte j of the 8 mantissa words a lane reads = column 4c+j), so the weights
//              are dequantised exactly once per workgroup and never written back to LDS as bf16
//   math       per k step a wavefront issues MB x 4 MFMAs (16x16x32) on 4 B operands; the VALU work of building
//              operand j+1 overlaps the MFMAs of operand j
// Semantics as in bfp_matmul.hip (tt::operations::primary::matmul, tt_eager/tt_dnn/op_library/bmm/bmm_op.hpp:318-346).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <type_traits>

#include "bfp_dequant.h"
#include "ttmi_internal.h"

namespace ttmi {

struct TileDev {
    const uint8_t *a;        // bf16
    const uint8_t *b;        // packed tiles
    const uint16_t *bias;    // bf16 [n] or null
    uint8_t *c;              // output (bf16 or fp32)
    uint32_t batch, b_batch, m, k, n;
    uint32_t kt, nt, tiles_m, tiles_n;
    int a_tiled, c_tiled, c_f32;
};

constexpr int TILE_STAGES = 4;
constexpr int TILE_COLS = 256;

template <int W, int ACT, int MB>
__global__ __launch_bounds__(256, 1) void matmul_tile_kernel(const TileDev p) {
    using F = Wfmt<W>;
    constexpr int BM = 16 * MB;
    constexpr int A_BYTES = BM * 64;                       // rows x 32 bf16
    constexpr int STAGE_BYTES = A_BYTES + 4 * F::stage_bytes;
    constexpr int NLOAD = F::loads;
    constexpr int A_LOADS = MB / 4;                        // direct-to-LDS loads of 16 rows each, per wavefront
    constexpr int VM_PER_STEP = NLOAD + A_LOADS;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[TILE_STAGES * STAGE_BYTES];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int t_of_lane = c >> 3, fc = (c >> 2) & 1, q = c & 3;
    const int h_of_lane = g >> 1, g_low = g & 1;

    // block coordinates: consecutive workgroups (which land on different XCDs) take different m blocks of the same
    // n block, so each XCD's L2 keeps re-serving one band of A while all of them stream the same weights
    uint32_t idx = blockIdx.x;
    const uint32_t tm = idx % p.tiles_m; idx /= p.tiles_m;
    const uint32_t tn = idx % p.tiles_n;
    const uint32_t bb = idx / p.tiles_n;
    const uint32_t m0 = tm * BM;
    const uint32_t nt0 = tn * (TILE_COLS / 32) + wave * 2;             // first packed tile column of this wavefront
    const uint32_t n_valid = nt0 >= p.nt ? 0u : min(2u, p.nt - nt0);

    // ---- where this lane's direct-to-LDS loads come from ----------------------------------------------------
    uint32_t chunk_of[NLOAD], src_off[NLOAD];
    stage_chunks<W>(lane, chunk_of);
    const uint32_t chunks_valid = (n_valid ? n_valid : 1u) * F::chunks;   // wavefronts past the edge reload tile 0 of the row
#pragma unroll
    for (int l = 0; l < NLOAD; ++l) src_off[l] = min(chunk_of[l], chunks_valid - 1) * 16;
    const uint32_t nt_src = n_valid ? nt0 : 0u;
    const uint8_t *wptr = p.b + ((uint64_t)(p.b_batch == 1 ? 0 : bb) * p.kt * p.nt + nt_src) * F::tile_bytes;
    const uint64_t w_step = (uint64_t)p.nt * F::tile_bytes;
    // A: load i of this wavefront brings rows wave*(BM/4) + i*16 + lane/4, 16 bytes at k offset (lane%4)*8
    uint32_t a_off[A_LOADS];
    const uint8_t *a_base;
    uint32_t a_step;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const uint32_t row_in_block = wave * (BM / 4) + i * 16 + (lane >> 2);
        const uint32_t row = min(m0 + row_in_block, p.m - 1);            // rows past M repeat the last row, never stored
        // the four 16-byte k chunks of a row are stored XOR-swizzled by (row / 4) % 4, so that the 16 lanes of one
        // ds_read_b128 pass (16 rows, same k chunk) hit 16 different 16-byte bank groups
        const uint32_t kq = (lane & 3) ^ ((lane >> 4) & 3);
        if (p.a_tiled) a_off[i] = (row >> 5) * p.kt * 2048 + (((row >> 4) & 1) * 2 + (kq >> 1)) * 512 + (row & 15) * 32 + (kq & 1) * 16;
        else a_off[i] = (row * p.k + kq * 8) * 2;
    }
    if (p.a_tiled) { a_base = p.a + (uint64_t)bb * ((p.m + 31) / 32) * p.kt * 2048; a_step = 2048; }
    else { a_base = p.a + (uint64_t)bb * p.m * p.k * 2; a_step = 64; }

    const uint32_t exp_off = A_BYTES + wave * F::stage_bytes + F::exp_base + t_of_lane * 64 + (2 * h_of_lane + fc) * 16 + g_low * 8;
    const uint32_t mant_off = A_BYTES + wave * F::stage_bytes + (h_of_lane * 4 + t_of_lane * 2 + fc) * F::face_stride +
                              (g_low * 8) * F::row_bytes + (W == 7 ? q * 4 : (q >> 1) * 4);
    const uint32_t a_read_off = c * 64 + ((g ^ ((c >> 2) & 3)) * 16);   // + mb * 1024: this lane's 16 bytes of the A operand

    auto fetch = [&](uint32_t stage) {
        uint8_t *base = lds + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(a_base + a_off[i]),
                                             (__attribute__((address_space(3))) void *)(base + (wave * (BM / 4) + i * 16) * 64), 16, 0, 0);
#pragma unroll
        for (int l = 0; l < NLOAD; ++l)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(wptr + src_off[l]),
                                             (__attribute__((address_space(3))) void *)(base + A_BYTES + wave * F::stage_bytes + l * 1024), 16, 0, 0);
        a_base += a_step;
        wptr += w_step;
    };

    f32x4 acc[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[mb][j][r] = 0.f;

    // Ring: k step i lives in stage i % TILE_STAGES and is requested TILE_STAGES - 1 steps ahead.  The loop is
    // software-pipelined inside the wavefront: while the MFMAs of step i run, the weights of step i+1 are expanded
    // into the other set of B operand registers.  Per iteration i:
    //   wait until this wavefront's share of step i+1 has landed; barrier (now every share of step i+1 has landed and
    //   every wavefront has finished reading step i-1, whose stage is refilled); read the packed words of step i+1;
    //   then for each 16-row block: read its A operand of step i from LDS (a window of A_WINDOW is kept in flight),
    //   issue its 4 MFMAs, and after every fourth of the blocks build one B operand of step i+1.
    const uint32_t total = p.kt;
    uint32_t requested = 0;
    for (; requested < total && requested < TILE_STAGES - 1; ++requested) fetch(requested);

    constexpr int A_WINDOW = 8;
    bf16x8 bop[2][4];
    StagedWords sw;
    uint32_t stage = 0, step = 0;      // the k step being multiplied and its stage
    auto wait_for_step = [&](uint32_t which) {       // vector-memory operations complete in order
        const uint32_t ahead = requested - which - 1;
        if (ahead >= 2) wait_vmcnt<2 * VM_PER_STEP>();
        else if (ahead == 1) wait_vmcnt<VM_PER_STEP>();
        else wait_vmcnt<0>();
    };
    // prologue: operands of step 0
    wait_for_step(0);
    __syncthreads();
    read_staged<W>(lds, exp_off, mant_off, sw);
    {
        float scale[8]; uint32_t mags[8];
        prepare_staged<W>(sw, q, scale, mags);
        bop[0][0] = weights_operand8<0>(sw.words, mags, scale);
        bop[0][1] = weights_operand8<1>(sw.words, mags, scale);
        bop[0][2] = weights_operand8<2>(sw.words, mags, scale);
        bop[0][3] = weights_operand8<3>(sw.words, mags, scale);
    }
    auto iteration = [&](auto cur_buf, auto has_next) {
        constexpr int C = decltype(cur_buf)::value, N = 1 - C;
        constexpr bool more = decltype(has_next)::value;
        const uint32_t next_stage = stage + 1 == TILE_STAGES ? 0 : stage + 1;
        const uint32_t a_at = stage * STAGE_BYTES + a_read_off;
        if (more) {
            wait_for_step(step + 1);
            __builtin_amdgcn_s_waitcnt(0xC07F);   // our LDS reads of the previous step have returned
            __syncthreads();
            if (requested < total) { fetch(stage == 0 ? TILE_STAGES - 1 : stage - 1); ++requested; }
        }
        bf16x8 aop[A_WINDOW];
#pragma unroll
        for (int mb = 0; mb < A_WINDOW; ++mb) aop[mb] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(lds + a_at + mb * 1024));
        if (more) read_staged<W>(lds, next_stage * STAGE_BYTES + exp_off, next_stage * STAGE_BYTES + mant_off, sw);
        float scale[8]; uint32_t mags[8];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[mb][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[mb % A_WINDOW], bop[C][j], acc[mb][j], 0, 0, 0);
            if (mb + A_WINDOW < MB) aop[mb % A_WINDOW] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(lds + a_at + (mb + A_WINDOW) * 1024));
            if (more) {
                constexpr int every = MB / 4;          // one operand of the next step per MB/4 row blocks
                if (mb == 0) prepare_staged<W>(sw, q, scale, mags);
                if (mb == every - 1) bop[N][0] = weights_operand8<0>(sw.words, mags, scale);
                if (mb == 2 * every - 1) bop[N][1] = weights_operand8<1>(sw.words, mags, scale);
                if (mb == 3 * every - 1) bop[N][2] = weights_operand8<2>(sw.words, mags, scale);
                if (mb == 4 * every - 1) bop[N][3] = weights_operand8<3>(sw.words, mags, scale);
            }
        }
        stage = next_stage;
        ++step;
    };
    using Buf0 = std::integral_constant<int, 0>;
    using Buf1 = std::integral_constant<int, 1>;
    // pairs of steps that both have a successor, then the last one or two steps; no branch inside a step touches
    // the accumulators
#pragma unroll 1
    while (step + 2 < total) {
        iteration(Buf0{}, std::true_type{});
        iteration(Buf1{}, std::true_type{});
    }
    if (total - step == 2) {
        iteration(Buf0{}, std::true_type{});
        iteration(Buf1{}, std::false_type{});
    } else {
        iteration(Buf0{}, std::false_type{});
    }

    // ---- epilogue: lane holds rows mb*16 + 4g + r, columns 4c .. 4c+3 of its wavefront's 64 ------------------
    if (t_of_lane >= (int)n_valid) return;
    const uint32_t n_col = (nt0 + t_of_lane) * 32 + fc * 16 + q * 4;
    float bias_v[4] = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
#pragma unroll
        for (int j = 0; j < 4; ++j) bias_v[j] = __uint_as_float((uint32_t)p.bias[n_col + j] << 16);
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t row = m0 + mb * 16 + g * 4 + r;
            if (row >= p.m) continue;
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = apply_activation<ACT>(acc[mb][j][r] + bias_v[j]);
            uint64_t elem;
            if (p.c_tiled) {
                const uint64_t tile = ((uint64_t)bb * ((p.m + 31) / 32) + (row >> 5)) * p.nt + nt0 + t_of_lane;
                elem = tile * 1024 + (((row >> 4) & 1) * 2 + fc) * 256 + (row & 15) * 16 + q * 4;
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
}

template <int W, int ACT, int MB>
static void launch_tile(const TileDev &p, uint32_t blocks, hipStream_t st) {
    hipLaunchKernelGGL((matmul_tile_kernel<W, ACT, MB>), dim3(blocks), dim3(256), 0, st, p);
}

template <int W, int MB>
static void launch_tile_act(const TileDev &p, int activation, uint32_t blocks, hipStream_t st) {
    switch (activation) {
        case TTMI_ACT_RELU: launch_tile<W, TTMI_ACT_RELU, MB>(p, blocks, st); break;
        case TTMI_ACT_GELU: launch_tile<W, TTMI_ACT_GELU, MB>(p, blocks, st); break;
        case TTMI_ACT_SILU: launch_tile<W, TTMI_ACT_SILU, MB>(p, blocks, st); break;
        default: launch_tile<W, TTMI_ACT_NONE, MB>(p, blocks, st); break;
    }
}

int matmul_bfp_tiled(const MatmulArgs &x, hipStream_t st) {
    TileDev p{};
    p.a = (const uint8_t *)x.a; p.b = (const uint8_t *)x.b; p.bias = (const uint16_t *)x.bias; p.c = (uint8_t *)x.c;
    p.batch = x.batch; p.b_batch = x.b_batch; p.m = x.m; p.k = x.k; p.n = x.n;
    p.kt = x.k / 32; p.nt = x.n / 32;
    p.a_tiled = x.a_layout == TTMI_TILE; p.c_tiled = x.c_layout == TTMI_TILE; p.c_f32 = x.c_dtype == TTMI_FLOAT32;
    // 256-row blocks when they fill the chip, 128-row blocks otherwise (fewer idle CUs, half the accumulators)
    const uint32_t tiles_n = (x.n + TILE_COLS - 1) / TILE_COLS;
    const uint64_t big = (uint64_t)x.batch * ((x.m + 255) / 256) * tiles_n;
    const char *force_bm = getenv("TTMI_MATMUL_BM");
    const bool use_256 = force_bm ? force_bm[0] == '2' : (x.m > 128 && big >= 256 && x.m % 256 == 0);
    const uint32_t bm = use_256 ? 256 : 128;
    p.tiles_m = (x.m + bm - 1) / bm; p.tiles_n = tiles_n;
    const uint64_t blocks = (uint64_t)x.batch * p.tiles_m * p.tiles_n;
    if (blocks > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: problem too large for one launch");
    if ((uint64_t)x.m * x.k * 2 > 0xffffffffull || (uint64_t)((x.m + 31) / 32) * p.kt * 2048 > 0xffffffffull)
        return fail(TTMI_ERR_UNSUPPORTED, "matmul: one batch slice of A exceeds 4 GiB");
    if ((reinterpret_cast<uintptr_t>(x.a) | reinterpret_cast<uintptr_t>(x.b) | reinterpret_cast<uintptr_t>(x.c)) & 15u)
        return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: a, b and c must be 16-byte aligned");
    if (x.b_fmt == TTMI_BFLOAT8_B) {
        if (use_256) launch_tile_act<7, 16>(p, x.activation, (uint32_t)blocks, st);
        else launch_tile_act<7, 8>(p, x.activation, (uint32_t)blocks, st);
    } else {
        if (use_256) launch_tile_act<3, 16>(p, x.activation, (uint32_t)blocks, st);
        else launch_tile_act<3, 8>(p, x.activation, (uint32_t)blocks, st);
    }
    return check_launch("matmul_tile_kernel");
}

}  // namespace ttmi
