// Tiled GEMM with block-float weights for gfx950, for tall activations (prefill, batched bmm): MFMA-bound.
//
// Two kernels share the staging and the weight expansion:
//   matmul_tile_kernel   4 wavefronts, (32*MB)-row x 256-column block of C; used with MB = 4 (128 rows) when 256-row
//                        blocks would leave CUs idle or M is not a multiple of 256, for long k ranges
//   matmul_tile8_kernel  8 wavefronts, 256 x 256 block (or 128 x 256, for short k ranges); the two wavefronts of a
//                        column group split the weight expansion and exchange operands through LDS (described at the kernel)
//   staging    the k loop advances one packed tile row (32 rows of W) at a time through a ring of LDS stages filled by
//              direct global->LDS loads
//   math       v_mfma_f32_32x32x16_bf16, fp32 accumulation
//   A          the block's rows x 32 k values of bf16 go to LDS as they lie in memory (64 bytes per row, the four
//              16-byte chunks of a row XOR-swizzled) and are shared by the wavefronts; the A operand of one MFMA
//              (32 rows x 16 k) is one ds_read_b128 per lane
//   W          a wavefront's 64 columns = 2 packed tiles per k step, staged in the layout of Wfmt and expanded straight
//              into B operands, never written back to LDS as packed data.  Lane (c = lane % 32, kh = lane / 32) reads,
//              for a 16-row slab s of the step, the 8 mantissa words of k rows 16s + 8kh .. + 7 that hold columns
//              4(c % 16) .. + 3; of each word it uses the two bytes 2(c / 16) and 2(c / 16) + 1: byte cb is its column
//              in 32-column operand cb.  Which 32 of the 64 columns an operand holds is therefore a permutation that
//              only the epilogue has to know.
// Semantics as in bfp_matmul.hip (tt::operations::primary::matmul, tt_eager/tt_dnn/op_library/bmm/bmm_op.hpp:318-346).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <type_traits>

#include "bfp_dequant.h"
#include "ttmi_internal.h"

namespace ttmi {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

struct TileDev {
    const uint8_t *a;        // bf16
    const uint8_t *b;        // packed tiles
    const uint16_t *bias;    // bf16 [n] or null
    uint8_t *c;              // output (bf16 or fp32)
    uint32_t batch, b_batch, m, k, n;
    uint32_t kt, nt, tiles_m, tiles_n;
    int a_tiled, c_tiled, c_f32;
    int c_bfp;               // 0, or the mantissa bits (7 | 3) of a block-float output in TILE layout
};

constexpr int TILE_STAGES = 4;
constexpr int TILE_COLS = 256;

// One 16-row slab of a staged pair of packed tiles, as read from LDS by one lane, and its expansion.
struct Slab { uint32_t e[8], words[8]; };

template <int W> __device__ __forceinline__ void read_slab(const uint8_t *lds, uint32_t exp_at, uint32_t mant_at, Slab &s) {
    using F = Wfmt<W>;
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) s.e[jj] = lds[exp_at + jj];
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) s.words[jj] = *reinterpret_cast<const uint32_t *>(lds + mant_at + jj * F::row_bytes);
}

// Row scales and mantissa-only words of a slab; `half_shift` = 16 * (c / 16) brings this lane's two columns to bytes 0, 1.
// The scale of a row is its exponent byte moved into the exponent field of a float: 2^(E - 127), i.e. 2^(bias_exp - 127)
// times too large for every row alike; the epilogue takes that power of two out of the sums again (exactly).  Rows with
// E = 0 are read as E = 1 (row_scale in bfp_dequant.h).
template <int W> __device__ __forceinline__ void prepare_slab(Slab &s, int q, uint32_t half_shift, float (&scale)[8], uint32_t (&mags)[8]) {
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) scale[jj] = row_scale(s.e[jj]);
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
        if (W == 7) {
            s.words[jj] >>= half_shift;
            mags[jj] = s.words[jj] & 0x7f7fu;
        } else {
            // four 4-bit codes -> one code per byte, sign bit moved from bit 3 to bit 7 of its byte
            uint32_t v = (s.words[jj] >> (16 * (q & 1))) & 0xffffu;
            v = (v | (v << 8)) & 0x00ff00ffu;
            v = ((v | (v << 4)) & 0x0f0f0f0fu) >> half_shift;
            s.words[jj] = v << 4;
            mags[jj] = v & 0x0707u;
        }
    }
}

template <int W, int ACT, int MB>
__global__ __launch_bounds__(256, 1) void matmul_tile_kernel(const TileDev p) {
    using F = Wfmt<W>;
    constexpr int BM = 32 * MB;
    constexpr int A_BYTES = BM * 64;                       // rows x 32 bf16
    constexpr int STAGE_BYTES = A_BYTES + 4 * F::stage_bytes;
    constexpr int NLOAD = F::loads;
    constexpr int A_LOADS = MB / 2;                        // direct-to-LDS loads of 16 rows each, per wavefront
    constexpr int VM_PER_STEP = NLOAD + A_LOADS;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[TILE_STAGES * STAGE_BYTES];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 31, kh = lane >> 5;                      // MFMA row / column index and k half of this lane
    const int c16 = c & 15, half = c >> 4;
    const int t_of_lane = c16 >> 3, fc = (c16 >> 2) & 1, q = c16 & 3;
    const uint32_t half_shift = 16 * half;

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
        // the four 16-byte k chunks of a row are stored XOR-swizzled by (row / 4) % 4, so that lanes reading the same
        // k chunk of consecutive rows hit different 16-byte bank groups
        const uint32_t kq = (lane & 3) ^ ((lane >> 4) & 3);
        if (p.a_tiled) a_off[i] = (row >> 5) * p.kt * 2048 + (((row >> 4) & 1) * 2 + (kq >> 1)) * 512 + (row & 15) * 32 + (kq & 1) * 16;
        else a_off[i] = (row * p.k + kq * 8) * 2;
    }
    if (p.a_tiled) { a_base = p.a + (uint64_t)bb * ((p.m + 31) / 32) * p.kt * 2048; a_step = 2048; }
    else { a_base = p.a + (uint64_t)bb * p.m * p.k * 2; a_step = 64; }

    // slab s of the step: k rows 16s + 8kh .. + 7 = rows 8kh .. of faces (h = s)
    const uint32_t exp_off = A_BYTES + wave * F::stage_bytes + F::exp_base + t_of_lane * 64 + fc * 16 + kh * 8;        // + s * 32
    const uint32_t mant_off = A_BYTES + wave * F::stage_bytes + (t_of_lane * 2 + fc) * F::face_stride +
                              (kh * 8) * F::row_bytes + (W == 7 ? q * 4 : (q >> 1) * 4);                                   // + s * 4 * face_stride
    // A operand of MFMA (row block rb, slab s): row rb*32 + c, 16-byte chunk 2s + kh of that row
    const uint32_t a_read_off0 = c * 64 + (((0 + kh) ^ ((c >> 2) & 3)) * 16);   // + rb * 2048
    const uint32_t a_read_off1 = c * 64 + (((2 + kh) ^ ((c >> 2) & 3)) * 16);

    auto fetch = [&](uint32_t stage) __attribute__((always_inline)) {
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

    f32x16 acc[MB][2];                                 // [32-row block][32-column operand]
#pragma unroll
    for (int rb = 0; rb < MB; ++rb)
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[rb][cb][r] = 0.f;

    // Ring: k step i lives in stage i % TILE_STAGES and is requested TILE_STAGES - 1 steps ahead.  The loop is
    // software-pipelined inside the wavefront: while the MFMAs of step i run, the weights of step i+1 are expanded
    // into the other set of B operand registers.  Per iteration i:
    //   wait until this wavefront's share of step i+1 has landed; barrier (now every share of step i+1 has landed and
    //   every wavefront has finished reading step i-1, whose stage is refilled); read the packed words of step i+1;
    //   then for each slab and 32-row block: read its A operand of step i from LDS (a window of them is kept in
    //   flight), issue its 2 MFMAs, and in between build the B operands of step i+1.
    const uint32_t total = p.kt;
    uint32_t requested = 0;
    for (; requested < total && requested < TILE_STAGES - 1; ++requested) fetch(requested);

    bf16x8 bop[2][2][2];               // [buffer][slab][operand]
    Slab slab[2];
    uint32_t stage = 0, step = 0;      // the k step being multiplied and its stage
    auto wait_for_step = [&](uint32_t which) __attribute__((always_inline)) {       // vector-memory operations complete in order
        const uint32_t ahead = requested - which - 1;
        if (ahead >= 2) wait_vmcnt<2 * VM_PER_STEP>();
        else if (ahead == 1) wait_vmcnt<VM_PER_STEP>();
        else wait_vmcnt<0>();
    };
    auto expand = [&](auto buf, auto which_slab) __attribute__((always_inline)) {
        constexpr int B = decltype(buf)::value, S = decltype(which_slab)::value;
        float scale[8]; uint32_t mags[8];
        prepare_slab<W>(slab[S], q, half_shift, scale, mags);
        bop[B][S][0] = weights_operand8<0>(slab[S].words, mags, scale);
        bop[B][S][1] = weights_operand8<1>(slab[S].words, mags, scale);
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    // prologue: operands of step 0
    wait_for_step(0);
    __syncthreads();
    read_slab<W>(lds, exp_off, mant_off, slab[0]);
    read_slab<W>(lds, exp_off + 32, mant_off + 4 * F::face_stride, slab[1]);
    expand(I0{}, I0{});
    expand(I0{}, I1{});

    auto iteration = [&](auto cur_buf, auto has_next) __attribute__((always_inline)) {
        constexpr int C = decltype(cur_buf)::value, N = 1 - C;
        constexpr bool more = decltype(has_next)::value;
        const uint32_t next_stage = stage + 1 == TILE_STAGES ? 0 : stage + 1;
        const uint32_t a_at0 = stage * STAGE_BYTES + a_read_off0, a_at1 = stage * STAGE_BYTES + a_read_off1;
        if (more) {
            wait_for_step(step + 1);
            // a bare barrier: __syncthreads() would also wait for every direct-to-LDS load still in flight (its
            // fence counts them as memory operations of this workgroup), and the ring lives on keeping them in flight
            __builtin_amdgcn_s_waitcnt(0xC07F);   // our LDS reads of the previous step have returned
            __builtin_amdgcn_s_barrier();
            if (requested < total) { fetch(stage == 0 ? TILE_STAGES - 1 : stage - 1); ++requested; }
        }
        // A operands in order of use: (slab 0, rb 0..MB-1), (slab 1, rb 0..MB-1); AW of them in flight
        constexpr int AW = 4, NA = 2 * MB;
        bf16x8 aop[AW];
        auto a_addr = [&](int i) { return (i < MB ? a_at0 : a_at1) + (uint32_t)(i % MB) * 2048u; };
#pragma unroll
        for (int i = 0; i < AW; ++i) aop[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(lds + a_addr(i)));
        if (more) {
            read_slab<W>(lds, next_stage * STAGE_BYTES + exp_off, next_stage * STAGE_BYTES + mant_off, slab[0]);
            read_slab<W>(lds, next_stage * STAGE_BYTES + exp_off + 32, next_stage * STAGE_BYTES + mant_off + 4 * F::face_stride, slab[1]);
        }
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const int s = i / MB, rb = i % MB;
            acc[rb][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aop[i % AW], bop[C][s][0], acc[rb][0], 0, 0, 0);
            acc[rb][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aop[i % AW], bop[C][s][1], acc[rb][1], 0, 0, 0);
            if (i + AW < NA) aop[i % AW] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(lds + a_addr(i + AW)));
            if (more) {
                if (i == NA / 4) expand(std::integral_constant<int, N>{}, I0{});
                if (i == (3 * NA) / 4) expand(std::integral_constant<int, N>{}, I1{});
            }
        }
        stage = next_stage;
        ++step;
    };
    // pairs of steps that both have a successor, then the last one or two steps; no branch inside a step touches
    // the accumulators
#pragma unroll 1
    while (step + 2 < total) {
        iteration(I0{}, std::true_type{});
        iteration(I1{}, std::true_type{});
    }
    if (total - step == 2) {
        iteration(I0{}, std::true_type{});
        iteration(I1{}, std::false_type{});
    } else {
        iteration(I0{}, std::false_type{});
    }

    // ---- epilogue: acc[rb][cb][i] is row rb*32 + (i/4)*8 + kh*4 + i%4, column 4*c16 + 2*half + cb of the wavefront's 64;
    // the ring is idle now and becomes the staging of store_wave_part (4 KB per 32 rows and wavefront)
    wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    StoreTarget o;
    o.c = p.c; o.bias = p.bias; o.m = p.m; o.n = p.n; o.nt = p.nt; o.slice = bb;
    o.row0 = m0; o.nt0 = nt0;
    o.unscale = F::unscale; o.c_tiled = p.c_tiled; o.c_f32 = p.c_f32; o.c_bfp = p.c_bfp;
    static_assert(MB == 4 && TILE_STAGES * STAGE_BYTES >= 4 * 16384, "the epilogue stages 128 rows x 64 columns per wavefront in the ring");
    store_wave_part<ACT>(acc, o, lds + wave * 16384, lane);
}

// ---------------------------------------------------------------------------------------------------------
// 256 x 256 block (MB = 4; MB = 2: 128 x 256) with EIGHT wavefronts (two per SIMD).  A single wavefront per SIMD cannot issue the weight
// expansion and the MFMAs of a 256-row block fast enough; two can, if the expansion is not done twice.  Wavefront
// (wc = w % 4, wr = w / 4) owns rows 32*MB*wr .. and columns 64*wc .. +63 of the block.  The two wavefronts of a
// column group share the work of expanding its weights: wr expands slab wr (k rows 16*wr .. +15) of the NEXT k step
// into bf16 B operands and leaves them in LDS, exactly as its lanes would hold them in registers; after the step's
// barrier both read all four operands of the group (2 slabs x 2 operands, one ds_read_b128 each).
//   LDS   ring of TILE_STAGES stages [A: 64*MB rows x 64 B][packed W: 4 column groups], then two operand buffers
//         [column group][slab][operand][lane] x 16 B (step parity)
//   step  wait for the own direct-to-LDS loads of step i+1, barrier, request step i+3, then interleaved:
//         (a) operands of step i and A from LDS -> 4*MB MFMAs (32x32x16), (b) expand slab wr of step i+1 -> LDS
template <int W, int ACT, int MB>                          // MB = 32-row blocks per wavefront: 4 (256-row block) or 2 (128-row block)
__global__ __launch_bounds__(512, 1) void matmul_tile8_kernel(const TileDev p) {
    using F = Wfmt<W>;
    constexpr int BM = 64 * MB;                            // rows of the block
    constexpr int A_BYTES = BM * 64;
    constexpr int STAGE_BYTES = A_BYTES + 4 * F::stage_bytes;
    constexpr int OPS_BYTES = 4 * 2 * 2 * 64 * 16;         // one operand buffer
    constexpr int OPS_BASE = TILE_STAGES * STAGE_BYTES;
    constexpr int NLOAD = F::loads;
    constexpr int W_LOADS0 = (NLOAD + 1) / 2, W_LOADS1 = NLOAD - W_LOADS0;   // packed-weight loads issued by wr = 0 / wr = 1
    constexpr int A_LOADS = MB / 2;                        // BM / 16 loads of 16 rows each over 8 wavefronts
    __shared__ __attribute__((aligned(1024))) uint8_t lds[OPS_BASE + 2 * OPS_BYTES];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wc = wave & 3, wr = wave >> 2;
    const int c = lane & 31, kh = lane >> 5;
    const int c16 = c & 15, half = c >> 4;
    const int t_of_lane = c16 >> 3, fc = (c16 >> 2) & 1, q = c16 & 3;
    const uint32_t half_shift = 16 * half;

    uint32_t idx = blockIdx.x;
    const uint32_t tm = idx % p.tiles_m; idx /= p.tiles_m;
    const uint32_t tn = idx % p.tiles_n;
    const uint32_t bb = idx / p.tiles_n;
    const uint32_t m0 = tm * BM;
    const uint32_t nt0 = tn * (TILE_COLS / 32) + wc * 2;               // first packed tile column of this column group
    const uint32_t n_valid = nt0 >= p.nt ? 0u : min(2u, p.nt - nt0);

    // ---- direct-to-LDS loads of this wavefront ---------------------------------------------------------------
    uint32_t chunk_of[NLOAD], src_off[NLOAD];
    stage_chunks<W>(lane, chunk_of);
    const uint32_t chunks_valid = (n_valid ? n_valid : 1u) * F::chunks;
#pragma unroll
    for (int l = 0; l < NLOAD; ++l) src_off[l] = min(chunk_of[l], chunks_valid - 1) * 16;
    const uint32_t nt_src = n_valid ? nt0 : 0u;
    const uint8_t *wptr = p.b + ((uint64_t)(p.b_batch == 1 ? 0 : bb) * p.kt * p.nt + nt_src) * F::tile_bytes;
    const uint64_t w_step = (uint64_t)p.nt * F::tile_bytes;
    uint32_t a_off[A_LOADS];
    const uint8_t *a_base;
    uint32_t a_step;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const uint32_t row_in_block = wave * (BM / 8) + i * 16 + (lane >> 2);
        const uint32_t row = min(m0 + row_in_block, p.m - 1);
        const uint32_t kq = (lane & 3) ^ ((lane >> 4) & 3);              // XOR swizzle of the row's four 16-byte chunks
        if (p.a_tiled) a_off[i] = (row >> 5) * p.kt * 2048 + (((row >> 4) & 1) * 2 + (kq >> 1)) * 512 + (row & 15) * 32 + (kq & 1) * 16;
        else a_off[i] = (row * p.k + kq * 8) * 2;
    }
    if (p.a_tiled) { a_base = p.a + (uint64_t)bb * ((p.m + 31) / 32) * p.kt * 2048; a_step = 2048; }
    else { a_base = p.a + (uint64_t)bb * p.m * p.k * 2; a_step = 64; }

    auto fetch = [&](uint32_t stage) __attribute__((always_inline)) {
        uint8_t *base = lds + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(a_base + a_off[i]),
                                             (__attribute__((address_space(3))) void *)(base + (wave * (BM / 8) + i * 16) * 64), 16, 0, 0);
        if (wr == 0) {
#pragma unroll
            for (int l = 0; l < W_LOADS0; ++l)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(wptr + src_off[l]),
                                                 (__attribute__((address_space(3))) void *)(base + A_BYTES + wc * F::stage_bytes + l * 1024), 16, 0, 0);
        } else {
#pragma unroll
            for (int l = W_LOADS0; l < NLOAD; ++l)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(wptr + src_off[l]),
                                                 (__attribute__((address_space(3))) void *)(base + A_BYTES + wc * F::stage_bytes + l * 1024), 16, 0, 0);
        }
        a_base += a_step;
        wptr += w_step;
    };

    // the slab this wavefront expands: slab wr = faces (h = wr), k rows 8kh .. of them
    const uint32_t exp_off = A_BYTES + wc * F::stage_bytes + F::exp_base + t_of_lane * 64 + fc * 16 + kh * 8 + wr * 32;
    const uint32_t mant_off = A_BYTES + wc * F::stage_bytes + (wr * 4 + t_of_lane * 2 + fc) * F::face_stride +
                              (kh * 8) * F::row_bytes + (W == 7 ? q * 4 : (q >> 1) * 4);
    const uint32_t ops_write_off = OPS_BASE + ((wc * 2 + wr) * 2) * 1024 + lane * 16;         // + parity * OPS_BYTES, + operand * 1024
    const uint32_t ops_partner_off = OPS_BASE + ((wc * 2 + (1 - wr)) * 2) * 1024 + lane * 16;  // the other slab's operands
    // A operand of MFMA (row block rb, slab s): row wr*32*MB + rb*32 + c, 16-byte chunk 2s + kh of that row (+ rb * 2048)
    const uint32_t a_own_off = (wr * 32 * MB + c) * 64 + (((2 * wr + kh) ^ ((c >> 2) & 3)) * 16);
    const uint32_t a_partner_off = (wr * 32 * MB + c) * 64 + (((2 * (1 - wr) + kh) ^ ((c >> 2) & 3)) * 16);

    f32x16 acc[MB][2];
#pragma unroll
    for (int rb = 0; rb < MB; ++rb)
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[rb][cb][r] = 0.f;

    const uint32_t total = p.kt;
    uint32_t requested = 0;
    for (; requested < total && requested < TILE_STAGES - 1; ++requested) fetch(requested);

    uint32_t stage = 0, step = 0;
    auto wait_for_step = [&](uint32_t which) __attribute__((always_inline)) {       // vector-memory operations complete in order
        const uint32_t ahead = which < requested ? requested - which - 1 : 0;
        if (wr == 0) {
            constexpr int VM = A_LOADS + W_LOADS0;
            if (ahead >= 2) wait_vmcnt<2 * VM>(); else if (ahead == 1) wait_vmcnt<VM>(); else wait_vmcnt<0>();
        } else {
            constexpr int VM = A_LOADS + W_LOADS1;
            if (ahead >= 2) wait_vmcnt<2 * VM>(); else if (ahead == 1) wait_vmcnt<VM>(); else wait_vmcnt<0>();
        }
    };
    // Expands slab wr of the step in `from_stage`: the operands stay in registers for this wavefront and go to operand
    // buffer `parity` for the other wavefront of the column group.
    auto expand = [&](uint32_t from_stage, uint32_t parity, bf16x8 (&ops)[2]) __attribute__((always_inline)) {
        Slab slab;
        read_slab<W>(lds, from_stage * STAGE_BYTES + exp_off, from_stage * STAGE_BYTES + mant_off, slab);
        float scale[8]; uint32_t mags[8];
        prepare_slab<W>(slab, q, half_shift, scale, mags);
        ops[0] = weights_operand8<0>(slab.words, mags, scale);
        ops[1] = weights_operand8<1>(slab.words, mags, scale);
        *reinterpret_cast<u32x4 *>(lds + parity * OPS_BYTES + ops_write_off) = __builtin_bit_cast(u32x4, ops[0]);
        *reinterpret_cast<u32x4 *>(lds + parity * OPS_BYTES + ops_write_off + 1024) = __builtin_bit_cast(u32x4, ops[1]);
    };
    auto read_a = [&](uint32_t from_stage, uint32_t off, bf16x8 (&a)[MB]) __attribute__((always_inline)) {
#pragma unroll
        for (int rb = 0; rb < MB; ++rb)
            a[rb] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(lds + from_stage * STAGE_BYTES + off + (uint32_t)rb * 2048u));
    };

    // prologue: own operands and own-slab A of step 0
    bf16x8 own[2], a_own[MB];
    wait_for_step(0);
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    expand(0, 0, own);
    read_a(0, a_own_off, a_own);

    // One k step.  Everything the first eight MFMAs need (own-slab operands, own-slab A) is already in registers when
    // the barrier opens; the other slab's operands and A arrive from LDS while those MFMAs run.  Then this
    // wavefront's slab of the next step is expanded, the second eight MFMAs follow, and the own-slab A of the next
    // step (in LDS since the barrier) is read ahead.
    auto iteration = [&](auto has_next) __attribute__((always_inline)) {
        constexpr bool more = decltype(has_next)::value;
        const uint32_t next_stage = stage + 1 == TILE_STAGES ? 0 : stage + 1;
        const uint32_t parity = step & 1;
        if (more) wait_for_step(step + 1);
        __builtin_amdgcn_s_waitcnt(0xC07F);   // our LDS reads and operand writes of the previous step are done
        __builtin_amdgcn_s_barrier();
        if (more && requested < total) { fetch(stage == 0 ? TILE_STAGES - 1 : stage - 1); ++requested; }
        bf16x8 part[2], a_part[MB];
        part[0] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(lds + parity * OPS_BYTES + ops_partner_off));
        part[1] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(lds + parity * OPS_BYTES + ops_partner_off + 1024));
        read_a(stage, a_partner_off, a_part);
#pragma unroll
        for (int rb = 0; rb < MB; ++rb) {
            acc[rb][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_own[rb], own[0], acc[rb][0], 0, 0, 0);
            acc[rb][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_own[rb], own[1], acc[rb][1], 0, 0, 0);
        }
        bf16x8 next_own[2];
        if (more) expand(next_stage, parity ^ 1, next_own);
#pragma unroll
        for (int rb = 0; rb < MB; ++rb) {
            acc[rb][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_part[rb], part[0], acc[rb][0], 0, 0, 0);
            acc[rb][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_part[rb], part[1], acc[rb][1], 0, 0, 0);
        }
        if (more) {
            read_a(next_stage, a_own_off, a_own);
            own[0] = next_own[0]; own[1] = next_own[1];
        }
        stage = next_stage;
        ++step;
    };
#pragma unroll 1
    while (step + 1 < total) iteration(std::true_type{});
    iteration(std::false_type{});

    // ---- epilogue: acc[rb][cb][i] is row wr*32*MB + rb*32 + (i/4)*8 + kh*4 + i%4, column 4*c16 + 2*half + cb of the group's 64;
    // the ring and the operand buffers are idle now and become the staging of store_wave_part (4 KB per 32 rows and wavefront)
    wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    StoreTarget o;
    o.c = p.c; o.bias = p.bias; o.m = p.m; o.n = p.n; o.nt = p.nt; o.slice = bb;
    o.row0 = m0 + wr * 32 * MB; o.nt0 = nt0;
    o.unscale = F::unscale; o.c_tiled = p.c_tiled; o.c_f32 = p.c_f32; o.c_bfp = p.c_bfp;
    static_assert(OPS_BASE + 2 * OPS_BYTES >= 8 * MB * 4096, "staging of the epilogue does not fit into LDS");
    store_wave_part<ACT>(acc, o, lds + wave * (MB * 4096), lane);
}

// ---------------------------------------------------------------------------------------------------------
// (32*NW)-row x 64-column block with NW wavefronts, one 32-row band each, for batched GEMMs whose row ranges are short
// and few (BERT-like bmm: 384 rows per slice): with 128 x 256 blocks such a problem occupies half the CUs with
// workgroups that expand every weight once per 128 rows.  Here a workgroup owns ALL rows of a slice for one 64-column
// group, so every weight is expanded once: wavefronts 0..7 each expand a quarter of a slab of the NEXT k step into the
// operand buffer (one wavefront expanding a whole slab makes the others wait for it at every barrier), and after the
// step's barrier every wavefront reads the four operands (2 slabs x 2).
//   A     nobody but its wavefront reads a band of 32 rows, so A goes from memory straight into registers in the layout of
//         the MFMA's A operand, six k steps ahead (a ring through LDS holds at most two to three steps of 24 KB in flight,
//         and with 1.5 to 2 us of latency that, not any pipe, set the step time)
//   LDS   ring of 6 stages [packed W of the group], then two operand buffers [step in pair][slab][operand][lane] x 16 B
//         (pair parity)
//   pair  two k steps per barrier: wait for the own loads of the next pair, barrier, operands of this pair from LDS ->
//         8 MFMAs (32x32x16); wavefronts 0..7 expand their parts of the next pair in between; request the steps 6 ahead
template <int W, int ACT, int NW>
__global__ __launch_bounds__(64 * NW, 1) void matmul_tall_kernel(const TileDev p) {
    using F = Wfmt<W>;
    constexpr int BM = 32 * NW;
    constexpr int D = 6;                                   // k steps requested ahead (A into registers, packed W into the ring)
    constexpr int STAGE_BYTES = F::stage_bytes;
    constexpr int OPS_BYTES = 2 * 2 * 2 * 64 * 16;         // one operand buffer: the two k steps of a pair
    constexpr int OPS_BASE = D * STAGE_BYTES;
    constexpr int LDS_BYTES = OPS_BASE + 2 * OPS_BYTES > NW * 4096 ? OPS_BASE + 2 * OPS_BYTES : NW * 4096;
    constexpr int NLOAD = F::loads;
    constexpr int W_LOADS0 = (NLOAD + 1) / 2, W_LOADS1 = NLOAD - W_LOADS0;   // packed-weight loads issued by wavefront 0 / 1
    constexpr int A_LOADS = 2;                             // one 16-byte load per lane and slab
    __shared__ __attribute__((aligned(1024))) uint8_t lds[LDS_BYTES];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 31, kh = lane >> 5;
    const int c16 = c & 15, half = c >> 4;
    const int t_of_lane = c16 >> 3, fc = (c16 >> 2) & 1, q = c16 & 3;
    const uint32_t half_shift = 16 * half;

    // workgroup i runs on XCD i % 8: every XCD gets a contiguous range of blocks, so that the column groups of a slice
    // (which all read the slice's A) share one L2
    uint32_t idx = blockIdx.x;
    if ((gridDim.x & 7u) == 0) idx = (idx & 7u) * (gridDim.x >> 3) + (idx >> 3);
    const uint32_t tm = idx % p.tiles_m; idx /= p.tiles_m;
    const uint32_t tn = idx % p.tiles_n;                                 // 64-column group
    const uint32_t bb = idx / p.tiles_n;
    const uint32_t m0 = tm * BM;
    const uint32_t nt0 = tn * 2;                                         // < nt
    const uint32_t n_valid = min(2u, p.nt - nt0);

    // ---- direct-to-LDS loads of this wavefront ---------------------------------------------------------------
    uint32_t chunk_of[NLOAD], src_off[NLOAD];
    stage_chunks<W>(lane, chunk_of);
    const uint32_t chunks_valid = n_valid * F::chunks;
#pragma unroll
    for (int l = 0; l < NLOAD; ++l) src_off[l] = min(chunk_of[l], chunks_valid - 1) * 16;
    const uint8_t *wptr = p.b + ((uint64_t)(p.b_batch == 1 ? 0 : bb) * p.kt * p.nt + nt0) * F::tile_bytes;
    const uint64_t w_step = (uint64_t)p.nt * F::tile_bytes;
    // A: a wavefront is the only reader of its 32 rows, so they go straight into registers in the layout of the MFMA's A
    // operand: lane (c, kh) holds, for slab s, the 16 bytes of row wave*32 + c at k chunk 2s + kh (in TILE layout the 64
    // lanes of such a load cover two whole faces)
    uint32_t a_off[A_LOADS];
    const uint8_t *a_base;
    uint32_t a_step;
    {
        const uint32_t row = min(m0 + wave * 32 + c, p.m - 1);           // rows past M repeat the last row, never stored
#pragma unroll
        for (int sl = 0; sl < A_LOADS; ++sl) {
            const uint32_t kq = 2 * sl + kh;
            if (p.a_tiled) a_off[sl] = (row >> 5) * p.kt * 2048 + (((row >> 4) & 1) * 2 + (kq >> 1)) * 512 + (row & 15) * 32 + (kq & 1) * 16;
            else a_off[sl] = (row * p.k + kq * 8) * 2;
        }
    }
    if (p.a_tiled) { a_base = p.a + (uint64_t)bb * ((p.m + 31) / 32) * p.kt * 2048; a_step = 2048; }
    else { a_base = p.a + (uint64_t)bb * p.m * p.k * 2; a_step = 64; }
    // The loads of A and the waits for them are inline assembly: with direct-to-LDS loads pending, the compiler's own
    // wait before the first use of a loaded register is for ALL vector-memory operations (seen here once per trip of the
    // loop, which emptied the six-step pipeline every six steps).  The ring registers are read-write operands of the
    // loads, so each entry stays in one physical register from request to use; vector-memory operations complete in
    // order, so wait_for_step() covers them.
    u32x4 a_ring[D][A_LOADS];
#pragma unroll
    for (int u = 0; u < D; ++u)
#pragma unroll
        for (int sl = 0; sl < A_LOADS; ++sl) a_ring[u][sl] = u32x4{0u, 0u, 0u, 0u};

    // requests of one k step: slot = step % D names both the registers for A and the ring stage for the packed weights
    auto fetch = [&](auto slot_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        uint8_t *base = lds + SLOT * STAGE_BYTES;
#pragma unroll
        for (int sl = 0; sl < A_LOADS; ++sl)
            asm volatile("global_load_dwordx4 %0, %1, %2" : "+v"(a_ring[SLOT][sl]) : "v"(a_off[sl]), "s"(a_base) : "memory");
        if (wave == 0) {
#pragma unroll
            for (int l = 0; l < W_LOADS0; ++l)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(wptr + src_off[l]),
                                                 (__attribute__((address_space(3))) void *)(base + l * 1024), 16, 0, 0);
        } else if (wave == 1) {
#pragma unroll
            for (int l = W_LOADS0; l < NLOAD; ++l)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(wptr + src_off[l]),
                                                 (__attribute__((address_space(3))) void *)(base + l * 1024), 16, 0, 0);
        }
        a_base += a_step;
        wptr += w_step;
    };

    // wavefront e = 0..7 expands a quarter of slab e / 4 (faces h = e / 4): of the 8 k rows 8kh .. that a lane holds of the
    // slab, rows 2pr and 2pr + 1 (pr = e % 4), i.e. one 32-bit word of each of the slab's two operands
    const int es = (wave >> 2) & 1, pr = wave & 3;
    const uint32_t exp_off = F::exp_base + t_of_lane * 64 + fc * 16 + kh * 8 + es * 32 + 2 * pr;
    const uint32_t mant_off = (es * 4 + t_of_lane * 2 + fc) * F::face_stride + (kh * 8 + 2 * pr) * F::row_bytes + (W == 7 ? q * 4 : (q >> 1) * 4);
    const uint32_t ops_write_off = OPS_BASE + (es * 2) * 1024 + lane * 16 + pr * 4;     // + parity * OPS_BYTES, + step in pair * 4096, + operand * 1024
    const uint32_t ops_read_off = OPS_BASE + lane * 16;                             // + parity * OPS_BYTES, + step in pair * 4096, + (slab * 2 + operand) * 1024
    f32x16 acc[1][2];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[0][cb][r] = 0.f;

    const uint32_t total = p.kt;
    uint32_t requested = 0, step = 0;
    using S0 = std::integral_constant<int, 0>; using S1 = std::integral_constant<int, 1>; using S2 = std::integral_constant<int, 2>;
    using S3 = std::integral_constant<int, 3>; using S4 = std::integral_constant<int, 4>; using S5 = std::integral_constant<int, 5>;
    static_assert(D == 6, "the request and iteration sequences below are written out for six slots");
    if (requested < total) { fetch(S0{}); ++requested; }
    if (requested < total) { fetch(S1{}); ++requested; }
    if (requested < total) { fetch(S2{}); ++requested; }
    if (requested < total) { fetch(S3{}); ++requested; }
    if (requested < total) { fetch(S4{}); ++requested; }
    if (requested < total) { fetch(S5{}); ++requested; }

    // vector-memory operations complete in order and every wavefront issues the same number per step (its two A loads
    // and its share of the weight loads), so "step `which` has landed" is a bound on the operations still in flight
    auto wait_for_step = [&](uint32_t which) __attribute__((always_inline)) {
        const uint32_t ahead = which < requested ? requested - which - 1 : 0;   // steps requested after `which`: 0 .. D - 1
        auto ladder = [&](auto vm_c) __attribute__((always_inline)) {
            constexpr int VM = decltype(vm_c)::value;
            if (ahead >= 5) wait_vmcnt<5 * VM>(); else if (ahead == 4) wait_vmcnt<4 * VM>(); else if (ahead == 3) wait_vmcnt<3 * VM>();
            else if (ahead == 2) wait_vmcnt<2 * VM>(); else if (ahead == 1) wait_vmcnt<VM>(); else wait_vmcnt<0>();
        };
        if (wave == 0) ladder(std::integral_constant<int, A_LOADS + W_LOADS0>{});
        else if (wave == 1) ladder(std::integral_constant<int, A_LOADS + W_LOADS1>{});
        else ladder(std::integral_constant<int, A_LOADS>{});
    };
    // wavefronts 0..7: expand their two rows of the step in `from_stage` into operand buffer `parity`; the arithmetic is
    // that of weights_operand8 for one pair of rows
    auto expand = [&](int from_stage, uint32_t ops_at) __attribute__((always_inline)) {
        const uint8_t *stage_at = lds + from_stage * STAGE_BYTES;
        const float scale0 = row_scale(stage_at[exp_off]), scale1 = row_scale(stage_at[exp_off + 1]);
        uint32_t word[2] = {*reinterpret_cast<const uint32_t *>(stage_at + mant_off), *reinterpret_cast<const uint32_t *>(stage_at + mant_off + F::row_bytes)};
        uint32_t mag[2];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            if (W == 7) {
                word[r] >>= half_shift;
                mag[r] = word[r] & 0x7f7fu;
            } else {                                         // four 4-bit codes -> one code per byte, sign to bit 7 of its byte
                uint32_t v = (word[r] >> (16 * (q & 1))) & 0xffffu;
                v = (v | (v << 8)) & 0x00ff00ffu;
                v = ((v | (v << 4)) & 0x0f0f0f0fu) >> half_shift;
                word[r] = v << 4;
                mag[r] = v & 0x0707u;
            }
        }
        const uint32_t both0 = __builtin_amdgcn_perm(__float_as_uint(byte_to_float<0>(mag[1]) * scale1),
                                                     __float_as_uint(byte_to_float<0>(mag[0]) * scale0), 0x07060302u);
        const uint32_t both1 = __builtin_amdgcn_perm(__float_as_uint(byte_to_float<1>(mag[1]) * scale1), __float_as_uint(byte_to_float<1>(mag[0]) * scale0), 0x07060302u);
        const uint32_t signs0 = __builtin_amdgcn_perm(word[1], word[0], (4u << 24) | (0x0cu << 16) | (0u << 8) | 0x0cu);
        const uint32_t signs1 = __builtin_amdgcn_perm(word[1], word[0], (5u << 24) | (0x0cu << 16) | (1u << 8) | 0x0cu);
        *reinterpret_cast<uint32_t *>(lds + ops_at + ops_write_off) = (signs0 & 0x80008000u) | both0;
        *reinterpret_cast<uint32_t *>(lds + ops_at + ops_write_off + 1024) = (signs1 & 0x80008000u) | both1;
    };

    // prologue: the operands of the first pair of steps
    wait_for_step(total > 1 ? 1 : 0);
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    if (wave < 8) {
        expand(0, 0);
        if (total > 1) expand(1, 4096);
    }

    // Two k steps per barrier (a step alone is 4 MFMAs per wavefront, too little for what a barrier and the loop around
    // it cost).  PAIR = (step / 2) % 3 names the slots 2 PAIR and 2 PAIR + 1; the second step of the last pair may not exist.
    auto iteration = [&](auto pair_c) __attribute__((always_inline)) {
        constexpr int FIRST = 2 * decltype(pair_c)::value, SECOND = FIRST + 1, NEXT0 = (FIRST + 2) % D, NEXT1 = (FIRST + 3) % D;
        const bool have1 = step + 1 < total, more0 = step + 2 < total, more1 = step + 3 < total;
        const uint32_t ops_now = ((step >> 1) & 1) * OPS_BYTES, ops_next = OPS_BYTES - ops_now;
        wait_for_step(more1 ? step + 3 : more0 ? step + 2 : have1 ? step + 1 : step);   // the next pair's weights; at the end at least this pair's A
        asm volatile("" : "+v"(a_ring[FIRST][0]), "+v"(a_ring[FIRST][1]), "+v"(a_ring[SECOND][0]), "+v"(a_ring[SECOND][1]) :: "memory");   // uses stay behind the wait
        __builtin_amdgcn_s_waitcnt(0xC07F);   // our LDS reads and operand writes of the previous pair are done
        __builtin_amdgcn_s_barrier();
        bf16x8 b[2][2][2];                    // [step in pair][slab][operand]
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int sb = 0; sb < 2; ++sb)
#pragma unroll
                for (int cb = 0; cb < 2; ++cb)
                    b[h][sb][cb] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(lds + ops_now + ops_read_off + h * 4096 + (sb * 2 + cb) * 1024));
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_ring[FIRST][0]), b[0][0][0], acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_ring[FIRST][0]), b[0][0][1], acc[0][1], 0, 0, 0);
        if (more0 && wave < 8) expand(NEXT0, ops_next);
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_ring[FIRST][1]), b[0][1][0], acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_ring[FIRST][1]), b[0][1][1], acc[0][1], 0, 0, 0);
        if (have1) {
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_ring[SECOND][0]), b[1][0][0], acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_ring[SECOND][0]), b[1][0][1], acc[0][1], 0, 0, 0);
        }
        if (more1 && wave < 8) expand(NEXT1, ops_next + 4096);
        if (have1) {
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_ring[SECOND][1]), b[1][1][0], acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_ring[SECOND][1]), b[1][1][1], acc[0][1], 0, 0, 0);
        }
        // the pair's registers and ring stages are free (the stages were read before the barrier above): request the
        // steps D ahead
        if (requested < total) { fetch(std::integral_constant<int, FIRST>{}); ++requested; }
        if (requested < total) { fetch(std::integral_constant<int, SECOND>{}); ++requested; }
        step += 2;
    };
#pragma unroll 1
    for (;;) {
        iteration(S0{}); if (step >= total) break;
        iteration(S1{}); if (step >= total) break;
        iteration(S2{}); if (step >= total) break;
    }

    // ---- epilogue: acc[0][cb][i] is row wave*32 + (i/4)*8 + kh*4 + i%4, column 4*c16 + 2*half + cb of the group's 64;
    // ring and operand buffers are idle now and become the staging of store_wave_part (4 KB per wavefront)
    wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    StoreTarget o;
    o.c = p.c; o.bias = p.bias; o.m = p.m; o.n = p.n; o.nt = p.nt; o.slice = bb;
    o.row0 = m0 + wave * 32; o.nt0 = nt0;
    o.unscale = F::unscale; o.c_tiled = p.c_tiled; o.c_f32 = p.c_f32; o.c_bfp = p.c_bfp;
    static_assert(LDS_BYTES >= NW * 4096, "staging of the epilogue does not fit into LDS");
    store_wave_part<ACT>(acc, o, lds + wave * 4096, lane);
}

template <int W, int NW>
static void launch_tall_act(const TileDev &p, int activation, uint32_t blocks, hipStream_t st) {
    switch (activation) {
        case TTMI_ACT_RELU: hipLaunchKernelGGL((matmul_tall_kernel<W, TTMI_ACT_RELU, NW>), dim3(blocks), dim3(64 * NW), 0, st, p); break;
        case TTMI_ACT_GELU: hipLaunchKernelGGL((matmul_tall_kernel<W, TTMI_ACT_GELU, NW>), dim3(blocks), dim3(64 * NW), 0, st, p); break;
        case TTMI_ACT_SILU: hipLaunchKernelGGL((matmul_tall_kernel<W, TTMI_ACT_SILU, NW>), dim3(blocks), dim3(64 * NW), 0, st, p); break;
        default: hipLaunchKernelGGL((matmul_tall_kernel<W, TTMI_ACT_NONE, NW>), dim3(blocks), dim3(64 * NW), 0, st, p); break;
    }
}

template <int W, int MB>
static void launch_tile8_act(const TileDev &p, int activation, uint32_t blocks, hipStream_t st) {
    switch (activation) {
        case TTMI_ACT_RELU: hipLaunchKernelGGL((matmul_tile8_kernel<W, TTMI_ACT_RELU, MB>), dim3(blocks), dim3(512), 0, st, p); break;
        case TTMI_ACT_GELU: hipLaunchKernelGGL((matmul_tile8_kernel<W, TTMI_ACT_GELU, MB>), dim3(blocks), dim3(512), 0, st, p); break;
        case TTMI_ACT_SILU: hipLaunchKernelGGL((matmul_tile8_kernel<W, TTMI_ACT_SILU, MB>), dim3(blocks), dim3(512), 0, st, p); break;
        default: hipLaunchKernelGGL((matmul_tile8_kernel<W, TTMI_ACT_NONE, MB>), dim3(blocks), dim3(512), 0, st, p); break;
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
    p.c_bfp = x.c_dtype == TTMI_BFLOAT8_B ? 7 : x.c_dtype == TTMI_BFLOAT4_B ? 3 : 0;
    // 256-row blocks when they fill the chip, 128-row blocks otherwise (fewer idle CUs, half the accumulators).
    // The test entry point can force a form (TTMI_KNOB_MATMUL_BLOCK): 256, 128 (eight wavefronts), 4 (128 rows, four wavefronts) or 384 (384 x 64).
    const uint32_t tiles_n = (x.n + TILE_COLS - 1) / TILE_COLS;
    const uint64_t big = (uint64_t)x.batch * ((x.m + 255) / 256) * tiles_n;
    uint32_t forced_form = 0;
    const bool force_bm = knob(TTMI_KNOB_MATMUL_BLOCK, &forced_form);
    // 384-row x 64-column blocks (every weight expanded once per slice) when the slices are whole multiples of 384 rows
    // and 128-row blocks would leave CUs without a workgroup
    constexpr int TALL_WAVES = 12;
    const uint64_t blocks_128 = (uint64_t)x.batch * ((x.m + 127) / 128) * tiles_n;
    const uint64_t blocks_tall = (uint64_t)x.batch * ((x.m + 32 * TALL_WAVES - 1) / (32 * TALL_WAVES)) * ((x.n + 63) / 64);
    const bool use_tall = force_bm ? forced_form == 384 : (x.m % (32 * TALL_WAVES) == 0 && blocks_128 < 256 && blocks_tall > blocks_128);
    if (use_tall) {
        p.tiles_m = (x.m + 32 * TALL_WAVES - 1) / (32 * TALL_WAVES); p.tiles_n = (x.n + 63) / 64;
        if (blocks_tall > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: problem too large for one launch");
        if ((uint64_t)x.m * x.k * 2 > 0xffffffffull || (uint64_t)((x.m + 31) / 32) * p.kt * 2048 > 0xffffffffull)
            return fail(TTMI_ERR_UNSUPPORTED, "matmul: one batch slice of A exceeds 4 GiB");
        if ((reinterpret_cast<uintptr_t>(x.a) | reinterpret_cast<uintptr_t>(x.b) | reinterpret_cast<uintptr_t>(x.c)) & 15u)
            return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: a, b and c must be 16-byte aligned");
        if (x.b_fmt == TTMI_BFLOAT8_B) launch_tall_act<7, TALL_WAVES>(p, x.activation, (uint32_t)blocks_tall, st);
        else launch_tall_act<3, TALL_WAVES>(p, x.activation, (uint32_t)blocks_tall, st);
        return check_launch("matmul_tall_kernel");
    }
    const bool use_256 = force_bm ? forced_form == 256 : (x.m > 128 && big >= 256 && x.m % 256 == 0);
    // 128-row blocks: eight wavefronts (each 64 rows) measure 6 % better than four for short k ranges (batched bmm,
    // k = 1024: epilogue and start-up are spread over twice as many wavefronts), four 1-2 % better for k = 4096
    const bool four_waves = force_bm ? forced_form == 4 : x.k > 2048;
    const uint32_t bm = use_256 ? 256 : 128;
    p.tiles_m = (x.m + bm - 1) / bm; p.tiles_n = tiles_n;
    const uint64_t blocks = (uint64_t)x.batch * p.tiles_m * p.tiles_n;
    if (blocks > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: problem too large for one launch");
    if ((uint64_t)x.m * x.k * 2 > 0xffffffffull || (uint64_t)((x.m + 31) / 32) * p.kt * 2048 > 0xffffffffull)
        return fail(TTMI_ERR_UNSUPPORTED, "matmul: one batch slice of A exceeds 4 GiB");
    if ((reinterpret_cast<uintptr_t>(x.a) | reinterpret_cast<uintptr_t>(x.b) | reinterpret_cast<uintptr_t>(x.c)) & 15u)
        return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: a, b and c must be 16-byte aligned");
    if (x.b_fmt == TTMI_BFLOAT8_B) {
        if (use_256) launch_tile8_act<7, 4>(p, x.activation, (uint32_t)blocks, st);
        else if (four_waves) launch_tile_act<7, 4>(p, x.activation, (uint32_t)blocks, st);
        else launch_tile8_act<7, 2>(p, x.activation, (uint32_t)blocks, st);
    } else {
        if (use_256) launch_tile8_act<3, 4>(p, x.activation, (uint32_t)blocks, st);
        else if (four_waves) launch_tile_act<3, 4>(p, x.activation, (uint32_t)blocks, st);
        else launch_tile8_act<3, 2>(p, x.activation, (uint32_t)blocks, st);
    }
    return check_launch("matmul_tile_kernel");
}

}  // namespace ttmi
