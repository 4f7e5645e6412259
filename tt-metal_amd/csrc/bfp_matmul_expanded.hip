// Two-pass GEMM with block-float weights for gfx950, for very tall activations (prefill): MFMA-bound.
//
// The fused kernels of bfp_matmul_tile.hip expand every packed weight once per 256-row block of C, and that expansion
// (vector ALU work) is what bounds them.  When many row blocks share the weights it is cheaper to expand them once:
//   expand_kernel            packed tiles -> bf16 values already in the register layout of MFMA B operands, written
//                            to a workspace in HBM (2 bytes per weight); HBM-bound
//   matmul_expanded_kernel   8 wavefronts, 256 x 256 block of C; A and the expanded weights go through an LDS ring filled
//                            by direct global->LDS loads; nothing but requests, LDS reads and
//                            v_mfma_f32_32x32x16_bf16 in the loop
// Workspace layout: [weight batch slice][k tile row][64-column group][slab s = k rows 16s..16s+15][operand cb][lane] x 16 B;
// lane (c = lane % 32, kh = lane / 32) holds k rows 16s + 8kh .. + 7 of the column that the fused kernels give it (see
// bfp_matmul_tile.hip), so both share the epilogue.  The values carry the common factor of Wfmt::unscale like there.
// Semantics as in bfp_matmul.hip (tt::operations::primary::matmul, tt_eager/tt_dnn/op_library/bmm/bmm_op.hpp:318-346).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <mutex>

#include "bfp_dequant.h"
#include "ttmi_internal.h"

namespace ttmi {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

constexpr int GROUP_BYTES = 4 * 1024;          // one k tile row of one 64-column group, expanded

// One wavefront per (k tile row, 64-column group): stage the 2 packed tiles in LDS in the layout of Wfmt, expand both
// 16-row slabs exactly as the fused kernels do, store 4 operands.
template <int W>
__global__ __launch_bounds__(256) void expand_kernel(const uint8_t *__restrict__ b, uint8_t *__restrict__ out, uint32_t kt,
                                                     uint32_t nt, uint32_t groups, uint32_t items) {
    using F = Wfmt<W>;
    constexpr int NLOAD = F::loads;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[4 * F::stage_bytes];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t item = blockIdx.x * 4 + wave;
    if (item >= items) return;                                   // no barrier in this kernel
    const uint32_t g = item % groups, row = item / groups;       // row = slice * kt + k tile row
    const uint32_t nt0 = g * 2, n_valid = min(2u, nt - nt0);
    const int c = lane & 31, kh = lane >> 5;
    const int c16 = c & 15, half = c >> 4;
    const int t_of_lane = c16 >> 3, fc = (c16 >> 2) & 1, q = c16 & 3;

    uint32_t chunk_of[NLOAD];
    stage_chunks<W>(lane, chunk_of);
    const uint8_t *src = b + ((uint64_t)row * nt + nt0) * F::tile_bytes;
    uint8_t *stage = lds + wave * F::stage_bytes;
#pragma unroll
    for (int l = 0; l < NLOAD; ++l)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + min(chunk_of[l], n_valid * F::chunks - 1) * 16),
                                         (__attribute__((address_space(3))) void *)(stage + l * 1024), 16, 0, 0);
    wait_vmcnt<0>();
    uint8_t *dst = out + (uint64_t)item * GROUP_BYTES + lane * 16;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        // slab s = faces with h = s, k rows 8kh .. 8kh + 7 of them
        const uint32_t exp_off = wave * F::stage_bytes + F::exp_base + t_of_lane * 64 + fc * 16 + kh * 8 + s * 32;
        const uint32_t mant_off = wave * F::stage_bytes + (s * 4 + t_of_lane * 2 + fc) * F::face_stride + (kh * 8) * F::row_bytes +
                                  (W == 7 ? q * 4 : (q >> 1) * 4);
        uint32_t e[8], words[8], mags[8];
        float scale[8];
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) e[jj] = lds[exp_off + jj];
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) words[jj] = *reinterpret_cast<const uint32_t *>(lds + mant_off + jj * F::row_bytes);
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) scale[jj] = row_scale(e[jj]);
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
            if (W == 7) {
                words[jj] >>= 16 * half;
                mags[jj] = words[jj] & 0x7f7fu;
            } else {
                uint32_t v = (words[jj] >> (16 * (q & 1))) & 0xffffu;
                v = (v | (v << 8)) & 0x00ff00ffu;
                v = ((v | (v << 4)) & 0x0f0f0f0fu) >> (16 * half);
                words[jj] = v << 4;
                mags[jj] = v & 0x0707u;
            }
        }
        const bf16x8 op0 = weights_operand8<0>(words, mags, scale), op1 = weights_operand8<1>(words, mags, scale);
        *reinterpret_cast<u32x4 *>(dst + (s * 2 + 0) * 1024) = __builtin_bit_cast(u32x4, op0);
        *reinterpret_cast<u32x4 *>(dst + (s * 2 + 1) * 1024) = __builtin_bit_cast(u32x4, op1);
    }
}

// The same workspace layout from bf16 weights in TILE layout (4-face tiles of 2048 bytes): a pure re-layout, so that a
// bf16 x bf16 GEMM (ttnn.matmul with two bf16 operands) runs on matmul_expanded_kernel too.  One wavefront per (k tile row,
// 64-column group): the 2 tiles go to LDS with 16 bytes per lane, and every lane gathers the 8 k rows of its column for the
// four operands.
__global__ __launch_bounds__(256) void relayout_bf16_kernel(const uint8_t *__restrict__ b, uint8_t *__restrict__ out, uint32_t nt, uint32_t groups,
                                                            uint32_t items) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[4 * 4096];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint32_t item = blockIdx.x * 4 + wave;
    if (item >= items) return;                                   // no barrier in this kernel
    const uint32_t g = item % groups, row = item / groups;       // row = slice * kt + k tile row
    const uint32_t nt0 = g * 2, n_valid = min(2u, nt - nt0);
    const int c = lane & 31, kh = lane >> 5;
    const int c16 = c & 15, half = c >> 4;
    const int t_of_lane = c16 >> 3, fc = (c16 >> 2) & 1, q = c16 & 3;
    const uint8_t *src = b + ((uint64_t)row * nt + nt0) * 2048;
    uint8_t *stage = lds + wave * 4096;
    // a tile past the matrix edge repeats the last one that exists (its columns are never stored by the GEMM)
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        const uint32_t chunk = l * 64 + lane;                     // 16-byte chunk of the 2 tiles
        const uint32_t tile = min(chunk >> 7, n_valid - 1);
        *reinterpret_cast<u32x4 *>(stage + chunk * 16) = *reinterpret_cast<const u32x4 *>(src + tile * 2048 + (chunk & 127) * 16);
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xC07F);                           // the wavefront's own LDS writes have landed
    uint8_t *dst = out + (uint64_t)item * GROUP_BYTES + lane * 16;
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) {
            // element (k row 16s + 8kh + i, column fc*16 + q*4 + half*2 + cb) of tile t_of_lane: face 2s + fc, 32 bytes per face row
            const uint32_t at = t_of_lane * 2048 + (2 * s + fc) * 512 + (8 * kh) * 32 + (q * 4 + half * 2 + cb) * 2;
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                w[i] = (uint32_t) * reinterpret_cast<const uint16_t *>(stage + at + (2 * i) * 32) |
                       ((uint32_t) * reinterpret_cast<const uint16_t *>(stage + at + (2 * i + 1) * 32) << 16);
            *reinterpret_cast<u32x4 *>(dst + (s * 2 + cb) * 1024) = u32x4{w[0], w[1], w[2], w[3]};
        }
}

struct ExpandedDev {
    const uint8_t *a;        // bf16
    const uint8_t *w;        // expanded weights (workspace)
    const uint16_t *bias;    // bf16 [n] or null
    uint8_t *c;
    uint32_t batch, b_batch, m, k, n;
    uint32_t kt, nt, groups, tiles_m, tiles_n, tiles_n8;
    float unscale;
    int a_tiled, c_tiled, c_f32;
    int c_bfp;               // 0, or the mantissa bits (7 | 3) of a block-float output in TILE layout
};

constexpr int EXP_STAGES = 4;

// 8 wavefronts, two per SIMD (while one issues LDS reads and requests the other issues MFMAs), each a 128 x 64 part of
// the 256 x 256 block: 4 x 2 accumulator blocks of 32 x 32.
//   LDS     ring of EXP_STAGES stages [A: 256 rows x 64 B, chunks XOR-swizzled][B: 4 column groups as they lie in the
//           workspace, 16 KB], both filled by direct global->LDS loads (4 per wavefront and step)
//   blocks  workgroup i runs on XCD i % 8.  An XCD takes every 8th 256-column block and all row blocks of it at the
//           same time, so a weight is fetched into one L2 only and A (small) is what every L2 re-reads.
//   step s  wait until everything requested before the previous step has landed (step s+1 complete in LDS), barrier,
//           then per 16-row slab 8 MFMAs, each followed by one LDS read of the following slab's operands (the first
//           slab of step s+1 at the end) or one request for step s+3.
template <int ACT>
__global__ __launch_bounds__(512, 1) void matmul_expanded_kernel(const ExpandedDev p) {
    constexpr int RB = 4, CB = 2;                          // 32-row and 32-column blocks per wavefront
    constexpr int A_BYTES = 256 * 64, B_BYTES = 4 * GROUP_BYTES;
    constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    constexpr int VM_PER_STEP = 4;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[EXP_STAGES * STAGE_BYTES];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wc = wave & 3, wr = wave >> 2;
    const int c = lane & 31, kh = lane >> 5;
    const uint32_t last = p.kt - 1;

    uint32_t idx = blockIdx.x;
    const uint32_t xcd = idx & 7; idx >>= 3;
    const uint32_t tm = idx % p.tiles_m; idx /= p.tiles_m;
    const uint32_t tn = (idx % p.tiles_n8) * 8 + xcd;
    const uint32_t bb = idx / p.tiles_n8;
    if (tn >= p.tiles_n) return;                                         // the whole workgroup, before any barrier
    const uint32_t m0 = tm * 256;

    // ---- requests of this wavefront: rows 32w .. 32w+31 of A, KB 2w, 2w+1 of the block's 16 KB of B -------------
    uint32_t a_off[2], b_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t row_in_block = wave * 32 + i * 16 + (lane >> 2);
        const uint32_t row = min(m0 + row_in_block, p.m - 1);
        const uint32_t kq = (lane & 3) ^ ((lane >> 4) & 3);              // XOR swizzle of the row's four 16-byte chunks
        if (p.a_tiled) a_off[i] = (row >> 5) * p.kt * 2048 + (((row >> 4) & 1) * 2 + (kq >> 1)) * 512 + (row & 15) * 32 + (kq & 1) * 16;
        else a_off[i] = (row * p.k + kq * 8) * 2;
        const uint32_t kb = wave * 2 + i;                                 // group kb / 4 of the block, KB kb % 4 of it
        const uint32_t group = min(tn * 4 + kb / 4, p.groups - 1);        // past the last group: any valid memory
        b_off[i] = group * GROUP_BYTES + (kb & 3) * 1024 + lane * 16;
    }
    const uint8_t *a_base;
    uint32_t a_step;
    if (p.a_tiled) { a_base = p.a + (uint64_t)bb * ((p.m + 31) / 32) * p.kt * 2048; a_step = 2048; }
    else { a_base = p.a + (uint64_t)bb * p.m * p.k * 2; a_step = 64; }
    const uint8_t *w_base = p.w + (uint64_t)(p.b_batch == 1 ? 0 : bb) * p.kt * p.groups * GROUP_BYTES;
    const uint64_t w_step = (uint64_t)p.groups * GROUP_BYTES;
    // request j of a step: j = 0, 1 the wavefront's A rows, j = 2, 3 its B KBs (steps past the end re-request the last one)
    auto request_one = [&](uint32_t kstep, int j) __attribute__((always_inline)) {
        uint8_t *stage = lds + (kstep & (EXP_STAGES - 1)) * STAGE_BYTES;
        const uint32_t at = min(kstep, last);
        const uint8_t *src = j < 2 ? a_base + (uint64_t)at * a_step + a_off[j] : w_base + at * w_step + b_off[j - 2];
        uint8_t *dst = j < 2 ? stage + (wave * 32 + j * 16) * 64 : stage + A_BYTES + (wave * 2 + (j - 2)) * 1024;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src, (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
    };
    auto request = [&](uint32_t kstep) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) request_one(kstep, j);
    };
    // operands of slab s: A of (row block rb) = row wr*128 + rb*32 + c, 16-byte chunk 2s + kh of that row;
    // B operand cb = KB wc*4 + 2s + cb of the stage's B
    uint32_t a_lds_off[2], b_lds_off[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        a_lds_off[s] = (wr * 128 + c) * 64 + (((2 * s + kh) ^ ((c >> 2) & 3)) * 16);
        b_lds_off[s] = A_BYTES + (wc * 4 + 2 * s) * 1024 + lane * 16;
    }
    // operand j of slab s: j = 0..3 the A operands (row blocks), j = 4, 5 the B operands
    auto read_operand = [&](uint32_t kstep, int s, int j, bf16x8 (&a)[RB], bf16x8 (&b)[CB]) __attribute__((always_inline)) {
        const uint32_t stage = (kstep & (EXP_STAGES - 1)) * STAGE_BYTES;
        if (j < 4) a[j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(lds + stage + a_lds_off[s] + (uint32_t)j * 2048u));
        else b[j - 4] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(lds + stage + b_lds_off[s] + (uint32_t)(j - 4) * 1024u));
    };

    f32x16 acc[RB][CB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[rb][cb][r] = 0.f;

    bf16x8 a0[RB], b0[CB], a1[RB], b1[CB], a2[RB], b2[CB];
    request(0); request(1); request(2);
    wait_vmcnt<VM_PER_STEP>();                 // steps 0 and 1 have landed (ours)
    __builtin_amdgcn_s_barrier();              // everybody's
#pragma unroll
    for (int j = 0; j < 6; ++j) read_operand(0, 0, j, a0, b0);

    // Between two MFMAs a wavefront issues at most one LDS read or one request (order of the reads: what the next slab
    // needs first), so that the matrix pipe never waits for a burst of them.  The operands of the next step's first
    // slab are read early in this step into a third set of registers: all wavefronts reach the barrier together, and
    // whatever they wait for there nobody hides.
    constexpr int read_order[6] = {0, 4, 5, 1, 2, 3};
    auto step_body = [&](uint32_t kstep, bf16x8 (&a_now)[RB], bf16x8 (&b_now)[CB], bf16x8 (&a_next)[RB], bf16x8 (&b_next)[CB]) __attribute__((always_inline)) {
        wait_vmcnt<VM_PER_STEP>();             // only the previous step's requests may still be in flight
        __builtin_amdgcn_s_waitcnt(0xC07F);    // our LDS reads of the previous step are done
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int i = 0; i < 8; ++i) {          // slab 0; reads of slab 1, then of slab 0 of the next step (in LDS since the barrier)
            acc[i >> 1][i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_now[i >> 1], b_now[i & 1], acc[i >> 1][i & 1], 0, 0, 0);
            if (i < 6) read_operand(kstep, 1, read_order[i], a1, b1);
            else read_operand(kstep + 1, 0, read_order[i - 6], a_next, b_next);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {          // slab 1; the remaining reads, then the requests for step + 3
            acc[i >> 1][i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1[i >> 1], b1[i & 1], acc[i >> 1][i & 1], 0, 0, 0);
            if (i < 4) read_operand(kstep + 1, 0, read_order[i + 2], a_next, b_next);
            else request_one(kstep + 3, i - 4);
            __builtin_amdgcn_sched_barrier(0);
        }
        asm volatile("" ::: "memory");         // the requests stay in this step
    };
    uint32_t kstep = 0;
#pragma unroll 1
    for (; kstep + 2 <= p.kt; kstep += 2) {
        step_body(kstep, a0, b0, a2, b2);
        step_body(kstep + 1, a2, b2, a0, b0);
    }
    if (kstep < p.kt) step_body(kstep, a0, b0, a2, b2);
    wait_vmcnt<0>();                           // requests past the end have landed,
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();              // and nobody reads operands any more: the ring becomes 8 x 16 KB of staging

    StoreTarget o;
    o.c = p.c; o.bias = p.bias; o.m = p.m; o.n = p.n; o.nt = p.nt; o.slice = bb;
    o.row0 = m0 + wr * 128; o.nt0 = (tn * 4 + wc) * 2;
    o.unscale = p.unscale; o.c_tiled = p.c_tiled; o.c_f32 = p.c_f32; o.c_bfp = p.c_bfp;
    store_wave_part<ACT>(acc, o, lds + wave * 16384, lane);
}

size_t matmul_expanded_workspace_bytes(uint32_t b_batch, uint32_t k, uint32_t n) {
    const uint64_t groups = ((uint64_t)n / 32 + 1) / 2;
    return (size_t)((uint64_t)b_batch * (k / 32) * groups * GROUP_BYTES);
}

// x.b: packed block-float tiles (x.b_fmt BFLOAT8_B | BFLOAT4_B) or bf16 tiles (x.b_fmt BFLOAT16)
int matmul_bfp_expanded(const MatmulArgs &x, hipStream_t st) {
    ExpandedDev p{};
    p.a = (const uint8_t *)x.a; p.bias = (const uint16_t *)x.bias; p.c = (uint8_t *)x.c;
    p.batch = x.batch; p.b_batch = x.b_batch; p.m = x.m; p.k = x.k; p.n = x.n;
    p.kt = x.k / 32; p.nt = x.n / 32; p.groups = (p.nt + 1) / 2;
    p.tiles_m = (x.m + 255) / 256; p.tiles_n = (x.n + 255) / 256; p.tiles_n8 = (p.tiles_n + 7) / 8;
    p.unscale = x.b_fmt == TTMI_BFLOAT8_B ? Wfmt<7>::unscale : x.b_fmt == TTMI_BFLOAT4_B ? Wfmt<3>::unscale : 1.0f;
    p.a_tiled = x.a_layout == TTMI_TILE; p.c_tiled = x.c_layout == TTMI_TILE; p.c_f32 = x.c_dtype == TTMI_FLOAT32;
    p.c_bfp = x.c_dtype == TTMI_BFLOAT8_B ? 7 : x.c_dtype == TTMI_BFLOAT4_B ? 3 : 0;
    const uint64_t blocks = (uint64_t)x.batch * p.tiles_m * p.tiles_n8 * 8;
    const uint64_t items = (uint64_t)x.b_batch * p.kt * p.groups;
    if (blocks > 0x7fffffffull || items > 0x7fffffffull) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: problem too large for one launch");
    if ((uint64_t)x.m * x.k * 2 > 0xffffffffull || (uint64_t)((x.m + 31) / 32) * p.kt * 2048 > 0xffffffffull)
        return fail(TTMI_ERR_UNSUPPORTED, "matmul: one batch slice of A exceeds 4 GiB");
    if ((reinterpret_cast<uintptr_t>(x.a) | reinterpret_cast<uintptr_t>(x.b) | reinterpret_cast<uintptr_t>(x.c)) & 15u)
        return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: a, b and c must be 16-byte aligned");
    const size_t need = matmul_expanded_workspace_bytes(x.b_batch, x.k, x.n);
    void *expanded = nullptr;
    if (x.workspace) {
        if (x.workspace_bytes < need) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: workspace of %zu bytes given, %zu needed", x.workspace_bytes, need);
        if (reinterpret_cast<uintptr_t>(x.workspace) & 255u) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: workspace must be 256-byte aligned");
        expanded = x.workspace;
    } else {
        // the library's own buffer, one per stream (launches on one stream run in order, so they can share it)
        bool fresh;
        if (int rc = scratch_get(SCRATCH_EXPANDED, st, need, &expanded, &fresh)) return rc;
    }
    p.w = (const uint8_t *)expanded;
    const uint32_t expand_blocks = (uint32_t)((items + 3) / 4);
    if (x.b_fmt == TTMI_BFLOAT8_B)
        hipLaunchKernelGGL((expand_kernel<7>), dim3(expand_blocks), dim3(256), 0, st, (const uint8_t *)x.b, (uint8_t *)expanded, p.kt, p.nt, p.groups, (uint32_t)items);
    else if (x.b_fmt == TTMI_BFLOAT4_B)
        hipLaunchKernelGGL((expand_kernel<3>), dim3(expand_blocks), dim3(256), 0, st, (const uint8_t *)x.b, (uint8_t *)expanded, p.kt, p.nt, p.groups, (uint32_t)items);
    else
        hipLaunchKernelGGL(relayout_bf16_kernel, dim3(expand_blocks), dim3(256), 0, st, (const uint8_t *)x.b, (uint8_t *)expanded, p.nt, p.groups, (uint32_t)items);
    if (int rc = check_launch("expand_kernel")) return rc;
    switch (x.activation) {
        case TTMI_ACT_RELU: hipLaunchKernelGGL((matmul_expanded_kernel<TTMI_ACT_RELU>), dim3((uint32_t)blocks), dim3(512), 0, st, p); break;
        case TTMI_ACT_GELU: hipLaunchKernelGGL((matmul_expanded_kernel<TTMI_ACT_GELU>), dim3((uint32_t)blocks), dim3(512), 0, st, p); break;
        case TTMI_ACT_SILU: hipLaunchKernelGGL((matmul_expanded_kernel<TTMI_ACT_SILU>), dim3((uint32_t)blocks), dim3(512), 0, st, p); break;
        default: hipLaunchKernelGGL((matmul_expanded_kernel<TTMI_ACT_NONE>), dim3((uint32_t)blocks), dim3(512), 0, st, p); break;
    }
    return check_launch("matmul_expanded_kernel");
}

}  // namespace ttmi
