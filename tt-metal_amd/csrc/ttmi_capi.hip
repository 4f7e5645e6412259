// The C ABI of libttmi: argument validation in the spirit of the reference's TT_FATAL checks, then a launch.
#include <stdarg.h>
#include <stdio.h>

#include "ttmi_internal.h"

namespace ttmi {

static thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char *what) {
    if (e == hipSuccess) return TTMI_OK;
    return fail(TTMI_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

int check_launch(const char *what) { return check_hip(hipGetLastError(), what); }

static bool is_bfp(int fmt) { return fmt == TTMI_BFLOAT8_B || fmt == TTMI_BFLOAT4_B; }

int validate_matmul(const void *a, int a_layout, const uint32_t *b, int b_fmt, uint32_t batch, uint32_t b_batch, uint32_t m, uint32_t k,
                    uint32_t n, int activation, const void *c, int c_layout, int c_dtype, bool allow_bf16_weights) {
    if (!is_bfp(b_fmt) && !(allow_bf16_weights && b_fmt == TTMI_BFLOAT16)) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: weight dtype must be BFLOAT8_B or BFLOAT4_B, got %d", b_fmt);
    if (!a || !b || !c) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: null pointer");
    if (batch == 0 || m == 0 || k == 0 || n == 0) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: empty dimension");
    // tt_eager/tt_dnn/op_library/bmm/multi_core_reuse_mcast_1d_optimized/...cpp:1207-1210: tile-multiple shapes
    if ((k & 31) || (n & 31)) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: K (%u) and N (%u) of the weights must be multiples of 32", k, n);
    if ((a_layout == TTMI_TILE || c_layout == TTMI_TILE) && (m & 31))
        return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: M (%u) must be a multiple of 32 for TILE layout", m);
    if ((a_layout != TTMI_TILE && a_layout != TTMI_ROW_MAJOR) || (c_layout != TTMI_TILE && c_layout != TTMI_ROW_MAJOR))
        return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: unknown layout");
    if (b_batch != 1 && b_batch != batch)
        return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: weight batch (%u) must be 1 or equal to the activation batch (%u)", b_batch, batch);
    if (c_dtype != TTMI_BFLOAT16 && c_dtype != TTMI_FLOAT32 && !is_bfp(c_dtype))
        return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: output dtype must be BFLOAT16, FLOAT32, BFLOAT8_B or BFLOAT4_B");
    if (is_bfp(c_dtype) && c_layout != TTMI_TILE) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: a block-float output needs TILE layout");
    if (activation < TTMI_ACT_NONE || activation > TTMI_ACT_SILU) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: unknown activation %d", activation);
    return TTMI_OK;
}

}  // namespace ttmi

using namespace ttmi;

extern "C" {

const char *ttmi_last_error(void) { return g_error; }
const char *ttmi_version(void) { return "ttmi 0.1 (gfx950)"; }

uint32_t ttmi_tile_size(int dtype) {
    switch (dtype) {
        case TTMI_BFLOAT8_B: return 1088;
        case TTMI_BFLOAT4_B: return 576;
        case TTMI_BFLOAT16: case TTMI_UINT16: return 2048;
        case TTMI_FLOAT32: case TTMI_UINT32: return 4096;
        default: return 0;
    }
}

size_t ttmi_tiled_size_bytes(int dtype, uint32_t batch, uint32_t h, uint32_t w) {
    const size_t ht = ((size_t)h + 31) / 32, wt = ((size_t)w + 31) / 32;
    return (size_t)batch * ht * wt * ttmi_tile_size(dtype);
}

int ttmi_pack_fp32_vec_as_bfp_tiles(int fmt, const float *src, size_t n_tiles, int row_major_input, uint32_t *dst,
                                    void *stream) {
    if (!is_bfp(fmt)) return fail(TTMI_ERR_INVALID_ARGUMENT, "pack: fmt must be BFLOAT8_B or BFLOAT4_B, got %d", fmt);
    if (n_tiles && (!src || !dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "pack: null pointer");
    return codec_pack_chunks(fmt, src, n_tiles, row_major_input, dst, (hipStream_t)stream);
}

int ttmi_unpack_bfp_tiles_into_float_vec(int fmt, const uint32_t *words, size_t n_tiles, int row_major_output,
                                         float *dst, void *stream) {
    if (!is_bfp(fmt)) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpack: fmt must be BFLOAT8_B or BFLOAT4_B, got %d", fmt);
    if (n_tiles && (!words || !dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpack: null pointer");
    return codec_unpack_chunks(fmt, words, n_tiles, row_major_output, dst, (hipStream_t)stream);
}

int ttmi_pack_rowmajor_as_bfp_tiles(int fmt, const void *src, int src_dtype, uint32_t batch, uint32_t h, uint32_t w,
                                    size_t row_stride, size_t batch_stride, uint32_t *dst, void *stream) {
    if (!is_bfp(fmt)) return fail(TTMI_ERR_INVALID_ARGUMENT, "pack: fmt must be BFLOAT8_B or BFLOAT4_B, got %d", fmt);
    if (src_dtype != TTMI_FLOAT32 && src_dtype != TTMI_BFLOAT16)
        return fail(TTMI_ERR_INVALID_ARGUMENT, "pack: source dtype must be FLOAT32 or BFLOAT16, got %d", src_dtype);
    if ((uint64_t)batch * h * w && (!src || !dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "pack: null pointer");
    if (row_stride < w || (batch > 1 && batch_stride < (size_t)h * row_stride))
        return fail(TTMI_ERR_INVALID_ARGUMENT, "pack: strides smaller than the extent they step over");
    return codec_pack_tensor(fmt, src, src_dtype == TTMI_FLOAT32 ? 4 : 2, batch, h, w, row_stride, batch_stride, dst,
                             (hipStream_t)stream);
}

int ttmi_unpack_bfp_tiles_as_rowmajor(int fmt, const uint32_t *words, uint32_t batch, uint32_t h, uint32_t w,
                                      void *dst, int dst_dtype, void *stream) {
    if (!is_bfp(fmt)) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpack: fmt must be BFLOAT8_B or BFLOAT4_B, got %d", fmt);
    if (dst_dtype != TTMI_FLOAT32 && dst_dtype != TTMI_BFLOAT16)
        return fail(TTMI_ERR_INVALID_ARGUMENT, "unpack: destination dtype must be FLOAT32 or BFLOAT16, got %d", dst_dtype);
    if ((uint64_t)batch * h * w && (!words || !dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpack: null pointer");
    return codec_unpack_tensor(fmt, words, batch, h, w, dst, dst_dtype == TTMI_FLOAT32 ? 4 : 2, (hipStream_t)stream);
}

int ttmi_tilize(const void *src, uint32_t elem_size, uint32_t batch, uint32_t h, uint32_t w, void *dst, void *stream) {
    if (elem_size != 2 && elem_size != 4) return fail(TTMI_ERR_INVALID_ARGUMENT, "tilize: element size must be 2 or 4, got %u", elem_size);
    if ((uint64_t)batch * h * w && (!src || !dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "tilize: null pointer");
    return codec_relayout(true, src, elem_size, batch, h, w, dst, (hipStream_t)stream);
}

int ttmi_untilize(const void *src, uint32_t elem_size, uint32_t batch, uint32_t h, uint32_t w, void *dst,
                  void *stream) {
    if (elem_size != 2 && elem_size != 4) return fail(TTMI_ERR_INVALID_ARGUMENT, "untilize: element size must be 2 or 4, got %u", elem_size);
    if ((uint64_t)batch * h * w && (!src || !dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "untilize: null pointer");
    return codec_relayout(false, src, elem_size, batch, h, w, dst, (hipStream_t)stream);
}

int ttmi_copy_window(int dtype, const void *src, const uint32_t src_shape[4], void *dst, const uint32_t dst_shape[4],
                     const int32_t offset[4], float fill, void *stream) {
    if (!src_shape || !dst_shape || !offset) return fail(TTMI_ERR_INVALID_ARGUMENT, "pad / unpad: null shape");
    uint64_t total = 1, src_total = 1;
    for (int d = 0; d < 4; ++d) { total *= dst_shape[d]; src_total *= src_shape[d]; }
    if (total && (!dst || (src_total && !src))) return fail(TTMI_ERR_INVALID_ARGUMENT, "pad / unpad: null pointer");
    return codec_copy_window(dtype, src, src_shape, dst, dst_shape, offset, fill, (hipStream_t)stream);
}

int ttmi_typecast_tiles(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n_tiles, void *stream) {
    if (n_tiles && (!src || !dst)) return fail(TTMI_ERR_INVALID_ARGUMENT, "typecast: null pointer");
    return codec_typecast_tiles(src, src_dtype, dst, dst_dtype, n_tiles, (hipStream_t)stream);
}

int ttmi_unpad_tiles(int dtype, const void *src, const uint32_t src_tiles[4], void *dst, const uint32_t start_tile[4],
                     const uint32_t dst_tiles[4], void *stream) {
    const uint32_t tile_bytes = ttmi_tile_size(dtype);
    if (!tile_bytes) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpad: unknown dtype %d", dtype);
    if (!src_tiles || !start_tile || !dst_tiles) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpad: null shape");
    if (!src || !dst) return fail(TTMI_ERR_INVALID_ARGUMENT, "unpad: null pointer");
    return codec_unpad_tiles(tile_bytes, src, src_tiles, dst, start_tile, dst_tiles, (hipStream_t)stream);
}

size_t ttmi_matmul_bfp_workspace_bytes(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt) {
    return matmul_workspace_bytes(batch, m, k, n, b_fmt);
}

size_t ttmi_matmul_bf16_workspace_bytes(uint32_t b_batch, uint32_t k, uint32_t n) {
    if (!b_batch || !k || !n) return 0;
    return matmul_expanded_workspace_bytes(b_batch, k, n);
}

int ttmi_matmul_bf16(const void *a, int a_layout, const void *b, uint32_t batch, uint32_t b_batch, uint32_t m, uint32_t k, uint32_t n,
                     const void *bias, int activation, void *c, int c_layout, int c_dtype, void *workspace, size_t workspace_bytes,
                     void *stream) {
    if (int rc = validate_matmul(a, a_layout, (const uint32_t *)b, TTMI_BFLOAT16, batch, b_batch, m, k, n, activation, c, c_layout, c_dtype, true)) return rc;
    MatmulArgs args{a, a_layout, (const uint32_t *)b, TTMI_BFLOAT16, batch, b_batch, m, k, n, bias, activation, c, c_layout, c_dtype, workspace, workspace_bytes};
    return matmul_bf16(args, (hipStream_t)stream);
}

int ttmi_matmul_bfp(const void *a, int a_layout, const uint32_t *b, int b_fmt, uint32_t batch, uint32_t b_batch,
                    uint32_t m, uint32_t k, uint32_t n, const void *bias, int activation, void *c, int c_layout,
                    int c_dtype, void *workspace, size_t workspace_bytes, void *stream) {
    if (int rc = validate_matmul(a, a_layout, b, b_fmt, batch, b_batch, m, k, n, activation, c, c_layout, c_dtype)) return rc;
    MatmulArgs args{a, a_layout, b, b_fmt, batch, b_batch, m, k, n, bias, activation, c, c_layout, c_dtype, workspace, workspace_bytes};
    return matmul_bfp(args, (hipStream_t)stream);
}

void ttmi_matmul_bfp_plan(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int a_dtype, int b_fmt, int c_dtype, uint32_t out[4]) {
    matmul_plan(batch, m, k, n, b_fmt, is_bfp(a_dtype) || is_bfp(c_dtype), out);
}

int ttmi_matmul_bfp_ab_supported(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int a_fmt, int b_fmt) {
    return a_fmt == TTMI_BFLOAT8_B && is_bfp(b_fmt) && (k & 31) == 0 && (n & 31) == 0 && matmul_takes_bfp_activations(batch, m, k, n, b_fmt) ? 1 : 0;
}

int ttmi_matmul_bfp_ab(const uint32_t *a, int a_fmt, const uint32_t *b, int b_fmt, uint32_t batch, uint32_t b_batch, uint32_t m, uint32_t k,
                       uint32_t n, const void *bias, int activation, void *c, int c_layout, int c_dtype, void *workspace,
                       size_t workspace_bytes, void *stream) {
    if (!is_bfp(a_fmt)) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: activation dtype must be BFLOAT8_B or BFLOAT4_B here, got %d", a_fmt);
    if (int rc = validate_matmul(a, TTMI_TILE, b, b_fmt, batch, b_batch, m, k, n, activation, c, c_layout, c_dtype)) return rc;
    if (a_fmt != TTMI_BFLOAT8_B)
        return fail(TTMI_ERR_UNSUPPORTED, "matmul: BFLOAT4_B activations are not taken by any kernel: expand them with ttmi_typecast_tiles first");
    MatmulArgs args{a, TTMI_TILE, b, b_fmt, batch, b_batch, m, k, n, bias, activation, c, c_layout, c_dtype, workspace, workspace_bytes};
    args.a_dtype = a_fmt;
    return matmul_bfp(args, (hipStream_t)stream);
}

size_t ttmi_matmul_bfp_gated_workspace_bytes(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt) {
    (void)b_fmt;
    return matmul_gated_workspace_bytes(batch, m, k, n);
}

int ttmi_matmul_bfp_gated(const void *a, int a_layout, const uint32_t *b_gate, const uint32_t *b_up, int b_fmt, uint32_t batch, uint32_t b_batch,
                          uint32_t m, uint32_t k, uint32_t n, const void *bias, int activation, void *c, int c_layout, int c_dtype,
                          void *workspace, size_t workspace_bytes, void *stream) {
    if (int rc = validate_matmul(a, a_layout, b_gate, b_fmt, batch, b_batch, m, k, n, activation, c, c_layout, c_dtype)) return rc;
    if (!b_up) return fail(TTMI_ERR_INVALID_ARGUMENT, "matmul: null pointer");
    MatmulArgs args{a, a_layout, b_gate, b_fmt, batch, b_batch, m, k, n, bias, activation, c, c_layout, c_dtype, workspace, workspace_bytes};
    args.b2 = b_up;
    return matmul_bfp_gated(args, (hipStream_t)stream);
}

int ttmi_eltwise_bf16(int op, const void *a, const void *b, float scalar, void *c, size_t count, void *stream) {
    if (count && (!a || !c)) return fail(TTMI_ERR_INVALID_ARGUMENT, "eltwise: null pointer");
    if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 15u)
        return fail(TTMI_ERR_INVALID_ARGUMENT, "eltwise: a, b and c must be 16-byte aligned");
    return eltwise_bf16(op, a, b, scalar, c, count, (hipStream_t)stream);
}

}  // extern "C"
