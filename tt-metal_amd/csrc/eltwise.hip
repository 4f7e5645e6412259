// Elementwise bf16 operations between the GEMMs of a block (HBM-bound: 6 B per element for a binary op, 4 B for a
// unary one).  Operands are flat arrays: TILE and ROW_MAJOR tensors of equal shape have equal element order, so the
// layout does not matter.  fp32 arithmetic, one round-to-nearest-even to bf16.
//   binary  tt::tt_metal::eltwise_binary (tt_eager/tt_dnn/op_library/eltwise_binary/eltwise_binary_op.hpp:20-38, 108-140)
//           as reached from ttnn.mul / ttnn.add / ttnn.sub (ttnn/ttnn/operations/binary.py:321-424)
//   unary   tt::tt_metal::eltwise_unary (tt_eager/tt_dnn/op_library/eltwise_unary/eltwise_unary_op.hpp:17-90): GELU, RELU, SILU
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bfp_dequant.h"
#include "ttmi_internal.h"

namespace ttmi {

template <int OP> __device__ __forceinline__ float eltwise_apply(float a, float b) {
    if (OP == TTMI_OP_ADD) return a + b;
    if (OP == TTMI_OP_SUB) return a - b;
    if (OP == TTMI_OP_MUL) return a * b;
    if (OP == TTMI_OP_GELU) return apply_activation<TTMI_ACT_GELU>(a);
    if (OP == TTMI_OP_RELU) return apply_activation<TTMI_ACT_RELU>(a);
    return apply_activation<TTMI_ACT_SILU>(a);
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// 8 elements (16 bytes) per lane and trip; `scalar` stands in for operand b when b is null (binary ops only)
template <int OP, bool BINARY>
__global__ __launch_bounds__(256) void eltwise_kernel(const uint16_t *a, const uint16_t *b, float scalar,
                                                      uint16_t *c, size_t count) {
    const size_t chunks = count / 8;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < chunks; i += (size_t)gridDim.x * blockDim.x) {
        const u32x4 va = reinterpret_cast<const u32x4 *>(a)[i];
        u32x4 vb = {0, 0, 0, 0};
        if (BINARY && b) vb = reinterpret_cast<const u32x4 *>(b)[i];
        u32x4 out;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float b0 = (BINARY && b) ? bf16_lo(vb[j]) : scalar, b1 = (BINARY && b) ? bf16_hi(vb[j]) : scalar;
            out[j] = f32x2_to_bf16x2_rne(eltwise_apply<OP>(bf16_lo(va[j]), b0), eltwise_apply<OP>(bf16_hi(va[j]), b1));
        }
        reinterpret_cast<u32x4 *>(c)[i] = out;
    }
    // the last count % 8 elements
    const size_t tail = chunks * 8 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tail < count) {
        const float x = __uint_as_float((uint32_t)a[tail] << 16);
        const float y = (BINARY && b) ? __uint_as_float((uint32_t)b[tail] << 16) : scalar;
        c[tail] = (uint16_t)f32x2_to_bf16x2_rne(eltwise_apply<OP>(x, y), 0.f);
    }
}

int eltwise_bf16(int op, const void *a, const void *b, float scalar, void *c, size_t count, hipStream_t st) {
    if (!count) return TTMI_OK;
    const size_t chunks = count / 8;
    size_t blocks = (chunks + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;          // 16 workgroups per CU, grid-stride beyond
    if (!blocks) blocks = 1;
    const uint16_t *pa = (const uint16_t *)a, *pb = (const uint16_t *)b;
    uint16_t *pc = (uint16_t *)c;
    switch (op) {
        case TTMI_OP_ADD: hipLaunchKernelGGL((eltwise_kernel<TTMI_OP_ADD, true>), dim3((uint32_t)blocks), dim3(256), 0, st, pa, pb, scalar, pc, count); break;
        case TTMI_OP_SUB: hipLaunchKernelGGL((eltwise_kernel<TTMI_OP_SUB, true>), dim3((uint32_t)blocks), dim3(256), 0, st, pa, pb, scalar, pc, count); break;
        case TTMI_OP_MUL: hipLaunchKernelGGL((eltwise_kernel<TTMI_OP_MUL, true>), dim3((uint32_t)blocks), dim3(256), 0, st, pa, pb, scalar, pc, count); break;
        case TTMI_OP_GELU: hipLaunchKernelGGL((eltwise_kernel<TTMI_OP_GELU, false>), dim3((uint32_t)blocks), dim3(256), 0, st, pa, pb, scalar, pc, count); break;
        case TTMI_OP_RELU: hipLaunchKernelGGL((eltwise_kernel<TTMI_OP_RELU, false>), dim3((uint32_t)blocks), dim3(256), 0, st, pa, pb, scalar, pc, count); break;
        case TTMI_OP_SILU: hipLaunchKernelGGL((eltwise_kernel<TTMI_OP_SILU, false>), dim3((uint32_t)blocks), dim3(256), 0, st, pa, pb, scalar, pc, count); break;
        default: return fail(TTMI_ERR_INVALID_ARGUMENT, "eltwise: unknown op %d", op);
    }
    return check_launch("eltwise_kernel");
}

}  // namespace ttmi
