/*
 * ttmi — block-float tensors on MI355X (gfx950): the C ABI.
 *
 * Every entry point is extern "C", takes plain pointers and sizes, returns an
 * int status (TTMI_OK == 0) and never throws.  ttmi_last_error() gives the
 * message of the last failure on the calling thread.  Unless a name says
 * "host", pointers are DEVICE pointers (hipMalloc'd memory of the current
 * device) and `stream` is a hipStream_t passed as void* (NULL = the null
 * stream).  Launches are asynchronous on that stream.
 *
 * Each declaration cites the tt-metal interface it stands in for (paths
 * relative to the tt-metal checkout).  The reference binds these through
 * pybind11 (tt_eager/tt_lib/csrc/tt_lib_bindings_tensor_pytensor.cpp and
 * ttnn/cpp/pybind11/operations/matmul.hpp); this C layer is what such a
 * binding would call.
 */
#ifndef TTMI_H
#define TTMI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TTMI_API __attribute__((visibility("default")))

/* status codes */
enum {
    TTMI_OK = 0,
    TTMI_ERR_INVALID_ARGUMENT = 1, /* what TT_FATAL / TT_THROW reject in the reference */
    TTMI_ERR_HIP = 2,              /* a HIP runtime call failed */
    TTMI_ERR_UNSUPPORTED = 3
};

/* tt_eager/tensor/types.hpp:26-34 DataType — same numeric values */
enum { TTMI_BFLOAT16 = 0, TTMI_FLOAT32 = 1, TTMI_UINT32 = 2, TTMI_BFLOAT8_B = 3, TTMI_BFLOAT4_B = 4, TTMI_UINT16 = 6 };

/* tt_eager/tensor/types.hpp:24 Layout — same numeric values */
enum { TTMI_ROW_MAJOR = 0, TTMI_TILE = 1 };

/* fused activation of ttnn.linear (ttnn/ttnn/operations/matmul.py:59-63) */
enum { TTMI_ACT_NONE = 0, TTMI_ACT_RELU = 1, TTMI_ACT_GELU = 2, TTMI_ACT_SILU = 3 };

/* elementwise operations of ttmi_eltwise_bf16: the binary ones carry the values of BinaryOpType
 * (tt_eager/tt_dnn/op_library/eltwise_binary/eltwise_binary_op.hpp:20-38), the unary ones 16 + TTMI_ACT_* */
enum { TTMI_OP_ADD = 0, TTMI_OP_SUB = 1, TTMI_OP_MUL = 2, TTMI_OP_RELU = 17, TTMI_OP_GELU = 18, TTMI_OP_SILU = 19 };

TTMI_API const char *ttmi_last_error(void);
TTMI_API const char *ttmi_version(void);

/* What kernels on the current device have reported since the last query: TTMI_OK, or TTMI_ERR_HIP (message in
 * ttmi_last_error()) when a matmul kernel gave up waiting for another workgroup's partial sums — the output of every
 * matmul launched on this device since the last query is then suspect (launches queued behind the one that gave up ran
 * on slots it left in disorder).
 * Reads a word of pinned host memory, no synchronisation; the report becomes visible once the kernel has run, and
 * ttmi_matmul_bfp makes the same check on entry.  The reference learns of a stuck kernel from its watcher thread
 * (tt_metal/impl/debug/watcher_server.cpp) or never; there is no call of this kind in it. */
TTMI_API int ttmi_device_status(void);

/* The library's own device memory.  A matmul called without a workspace takes its scratch — partial-sum slots, or the
 * weights expanded to bf16 (2 bytes per weight) — from a buffer that the library allocates on first use and keeps, one per
 * purpose, device and stream (launches on different streams may overlap and never share one); a buffer that has become
 * too small is replaced by one at least twice its size and kept aside until now.  Nothing is freed while the process runs
 * unless this is called: it waits for the current device to go idle (hipDeviceSynchronize) and frees every buffer that the
 * library holds on it, so a caller that has created many streams, or is done with large shapes, gets the memory back; the
 * next call without a workspace allocates again.  Returns the number of bytes freed through *freed_bytes (may be NULL).
 * No counterpart in the reference, whose allocator owns all device memory (tt_metal/impl/allocator). */
TTMI_API int ttmi_release_scratch(size_t *freed_bytes);

/* tt_metal/common/tt_backend_api_types.hpp:109-132 tile_size(DataFormat): bytes of one 32x32 tile
 * (1088 bfloat8_b, 576 bfloat4_b, 2048 bfloat16/uint16, 4096 float32/uint32); 0 for an unknown dtype. */
TTMI_API uint32_t ttmi_tile_size(int dtype);

/* tt_eager/tensor/tensor_utils.hpp:33-49 compute_buffer_size: bytes of a [batch, h, w] tensor in TILE layout
 * after h and w are rounded up to 32 (ttnn/ttnn/operations/core.py:793 pads with zeros). */
TTMI_API size_t ttmi_tiled_size_bytes(int dtype, uint32_t batch, uint32_t h, uint32_t w);

/* tt_metal/common/bfloat8.hpp:102 pack_fp32_vec_as_bfp8_tiles and bfloat4.hpp:23 pack_fp32_vec_as_bfp4_tiles
 * (is_exp_a = false).  src: n_tiles*1024 fp32, each 1024-chunk a row-major 32x32 block (row_major_input != 0)
 * or already in 4-face order.  dst: n_tiles * tile_size/4 words.  fmt: TTMI_BFLOAT8_B | TTMI_BFLOAT4_B. */
TTMI_API int ttmi_pack_fp32_vec_as_bfp_tiles(int fmt, const float *src, size_t n_tiles, int row_major_input, uint32_t *dst,
                                    void *stream);

/* bfloat8.hpp:175 unpack_bfp8_tiles_into_float_vec and bfloat4.hpp:33 unpack_bfp4_tiles_into_float_vec
 * (is_exp_a = false): inverse of the above, fp32 out. */
TTMI_API int ttmi_unpack_bfp_tiles_into_float_vec(int fmt, const uint32_t *words, size_t n_tiles, int row_major_output,
                                         float *dst, void *stream);

/* The whole host sequence of ttnn.from_torch(dtype=bfloat8_b|bfloat4_b, layout=TILE_LAYOUT) in one pass
 * (ttnn/ttnn/operations/core.py:276-309, tt_lib_bindings_tensor_pytensor.cpp:78-151,
 * tt_eager/tensor/tensor_impl.cpp:179-197): zero-pad h, w to 32, tilize to 4-face tiles, pack.
 * src: [batch, h, w] row-major, src_dtype TTMI_FLOAT32 or TTMI_BFLOAT16; consecutive rows are `row_stride`
 * elements apart (pass w for a dense tensor) and consecutive [h, w] slices batch_stride elements apart
 * (pass h*row_stride).  dst: ttmi_tiled_size_bytes(fmt, batch, h, w) bytes. */
TTMI_API int ttmi_pack_rowmajor_as_bfp_tiles(int fmt, const void *src, int src_dtype, uint32_t batch, uint32_t h, uint32_t w,
                                    size_t row_stride, size_t batch_stride, uint32_t *dst, void *stream);

/* The whole host sequence of ttnn.to_torch for a block-float tensor (core.py:336-394, tensor_impl.cpp:179-197,
 * tt_lib_bindings_tensor_pytensor.cpp:382-393): unpack, untilize, drop the tile padding.
 * words: tiles of the padded tensor.  dst: dense [batch, h, w] row-major, dst_dtype TTMI_FLOAT32 (what the
 * reference returns) or TTMI_BFLOAT16 (exact: unpacked values carry at most 7 significant bits). */
TTMI_API int ttmi_unpack_bfp_tiles_as_rowmajor(int fmt, const uint32_t *words, uint32_t batch, uint32_t h, uint32_t w,
                                      void *dst, int dst_dtype, void *stream);

/* tt_metal/common/test_tiles.hpp:177 convert_layout(LIN_ROW_MAJOR -> TILED32_4FACES), which is what
 * Tensor::to(Layout::TILE) runs (tt_eager/tensor/tensor_impl.hpp:158-165), and
 * tt_metal/common/tilize_untilize.hpp:9 tilize.  elem_size 2 or 4.  src [batch, h, w] dense row-major;
 * dst holds the zero-padded tensor in tile order. */
TTMI_API int ttmi_tilize(const void *src, uint32_t elem_size, uint32_t batch, uint32_t h, uint32_t w, void *dst, void *stream);

/* test_tiles.hpp:177 convert_layout(TILED32_4FACES -> LIN_ROW_MAJOR) (tensor_impl.hpp:167-171) and
 * tilize_untilize.hpp:68 untilize.  src: tiles of the padded tensor; dst: dense [batch, h, w] (padding dropped). */
TTMI_API int ttmi_untilize(const void *src, uint32_t elem_size, uint32_t batch, uint32_t h, uint32_t w, void *dst,
                  void *stream);

/* Tensor::pad and Tensor::unpad on 4-D row-major data (tt_eager/tensor/tensor.cpp:204-260 -> tt_eager/tensor/tensor_impl.hpp:508-578
 * pad<T>, :609-660 unpad<T>), and for block-float tensors pad_bfloat8_b / unpad_bfloat8_b / pad_bfloat4_b / unpad_bfloat4_b
 * (tt_eager/tensor/tensor_impl.cpp:200-283: unpack the sequential 1024-element chunks, pad or unpad as fp32, pack again),
 * in one pass:  dst[i0,i1,i2,i3] = src[i0-o0, i1-o1, i2-o2, i3-o3] where that index lies inside src, `fill` elsewhere.
 *   pad    offset = input_tensor_start, dst_shape = output_tensor_shape, fill = pad_value
 *   unpad  offset = -output_tensor_start, dst_shape = output_tensor_end - output_tensor_start + 1
 * dtype: TTMI_FLOAT32 | TTMI_UINT32 | TTMI_BFLOAT16 | TTMI_UINT16 (dense elements; fill is converted as static_cast<T>
 * does in the reference: a bfloat16 keeps the upper 16 bits of the float), or TTMI_BFLOAT8_B | TTMI_BFLOAT4_B (src and dst
 * are packed words of tensors declared ROW_MAJOR; both volumes must be multiples of 1024, both pointers 16-byte aligned). */
TTMI_API int ttmi_copy_window(int dtype, const void *src, const uint32_t src_shape[4], void *dst, const uint32_t dst_shape[4],
                     const int32_t offset[4], float fill, void *stream);

/* tt::tt_metal::typecast / clone(output_dtype) on a device tensor in TILE layout (tt_eager/tt_dnn/op_library/copy/copy_op.hpp:42-44;
 * also what tilize(output_dtype) and a block-float matmul output do, tt_eager/tt_dnn/op_library/tilize/tilize_op.hpp:71-73):
 * n_tiles tiles of 1024 elements in 4-face order change their data type, element order unchanged, in one pass.
 * Supported: BFLOAT16 | FLOAT32 -> BFLOAT8_B | BFLOAT4_B (the arithmetic of the host packers, one shared exponent per
 * 16-element face row), BFLOAT8_B | BFLOAT4_B -> BFLOAT16 | FLOAT32 (exact: at most 7 significant bits), BFLOAT16 -> FLOAT32
 * (exact) and FLOAT32 -> BFLOAT16 (round to nearest even).  The rounding of the Tensix packer that the reference's device op
 * uses is not in its sources (it lives in the LLK submodules): parity with the device op itself is unpinned. */
TTMI_API int ttmi_typecast_tiles(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n_tiles, void *stream);

/* tt::tt_metal::unpad on a device tensor in TILE layout (tt_eager/tt_dnn/op_library/unpad/unpad_op.hpp:14-40, the op behind
 * ttnn.Tensor.__getitem__, ttnn/ttnn/operations/core.py:99-108): start and end are tile-aligned there
 * (unpad_op.cpp validate), so whole tiles move and a block-float tensor keeps its codes.
 * src: tiles of a tensor whose tile grid is src_tiles = [N, C, H/32, W/32] (tile (n, c, r, q) at ((n*C + c)*Ht + r)*Wt + q);
 * dst: the dst_tiles grid that starts at start_tile.  dtype gives the tile size. */
TTMI_API int ttmi_unpad_tiles(int dtype, const void *src, const uint32_t src_tiles[4], void *dst, const uint32_t start_tile[4],
                     const uint32_t dst_tiles[4], void *stream);

/* Bytes of scratch ttmi_matmul_bfp wants for these sizes (0 when none).  No reference counterpart: the
 * reference's op allocates its circular buffers inside the program factory
 * (tt_eager/tt_dnn/op_library/bmm/multi_core_reuse_mcast_1d_optimized/bmm_op_multi_core_reuse_mcast_1d_optimized.cpp:48-52). */
TTMI_API size_t ttmi_matmul_bfp_workspace_bytes(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt);

/* C[b, m, n] = act(A[b, m, k] . B[(b | 0), k, n] + bias[n]) with block-float weights:
 * tt::operations::primary::matmul (tt_eager/tt_dnn/op_library/bmm/bmm_op.hpp:318-346, validate
 * bmm_op.cpp:828-1049) as reached from ttnn.matmul / ttnn.linear (ttnn/cpp/ttnn/operations/matmul.hpp:44-214)
 * and tt_lib.tensor.matmul / bmm (bmm_op.hpp:388-456).
 *   a        bf16, [batch, m, k]; a_layout TTMI_ROW_MAJOR (dense) or TTMI_TILE (4-face tiles, tile (mt, kt) of
 *            slice b at index (b*Mt + mt)*Kt + kt; m, k multiples of 32)
 *   b        packed tiles, b_fmt TTMI_BFLOAT8_B | TTMI_BFLOAT4_B, tile (kt, nt) at index kt*Nt + nt, k and n
 *            multiples of 32; b_batch is `batch` (bmm) or 1 (weights broadcast over the batch: bcast_batch)
 *   bias     NULL or bf16 [n] (row-broadcast add, matmul.hpp:117-214)
 *   c        c_dtype TTMI_BFLOAT16 (round to nearest even) or TTMI_FLOAT32; c_layout as for a.  Or c_dtype TTMI_BFLOAT8_B |
 *            TTMI_BFLOAT4_B with c_layout TTMI_TILE (output_dtype of tt::operations::primary::matmul, bmm_op.hpp:318-346):
 *            packed tiles of the bf16-rounded result with the host packers' arithmetic (what ttmi_typecast_tiles gives for
 *            the bf16 output), packed in the epilogue of whichever kernel the shape goes to: one launch, no buffer in between
 *   workspace NULL (the library keeps a buffer of its own per device and stream, allocated on first use) or at least
 *            ttmi_matmul_bfp_workspace_bytes() bytes of device memory, 256-byte aligned.  Where the weights are streamed
 *            (up to 127 rows, and taller activations whose output has too few blocks to fill the chip) it holds partial
 *            sums of workgroups that share an output (a few MB); where they are expanded to bf16 first (from 512 rows
 *            on), the expanded weights (2 bytes per weight; the size query assumes every batch slice has weights of its
 *            own, a call with b_batch == 1 needs only one slice's worth)
 * fp32 accumulation throughout. */
TTMI_API int ttmi_matmul_bfp(const void *a, int a_layout, const uint32_t *b, int b_fmt, uint32_t batch, uint32_t b_batch,
                    uint32_t m, uint32_t k, uint32_t n, const void *bias, int activation, void *c, int c_layout,
                    int c_dtype, void *workspace, size_t workspace_bytes, void *stream);

/* The same GEMM with block-float ACTIVATIONS (tt_eager/tt_dnn/op_library/bmm/bmm_op.cpp:531,839 accept BFLOAT8_B for input a;
 * tests/ttnn/unit_tests/operations/test_matmul.py:561-620 multiplies two BFLOAT8_B tensors):
 *   a        packed BFLOAT8_B tiles, tile (mt, kt) of slice s at index (s*Mt + mt)*Kt + kt; m a multiple of 32
 * The kernel that streams the weights expands the activations itself — exactly, to the bf16 values ttmi_typecast_tiles gives —
 * so the result is bit for bit that of ttmi_typecast_tiles(a -> BFLOAT16) followed by ttmi_matmul_bfp (but for face rows
 * of A with exponent byte 0, values below 2^-126, which the kernel reads with the scale of exponent 1 as it reads such
 * rows of the weights), in one launch and
 * with no bf16 copy of A (Falcon-7B 4h_to_h, M = 32: 23.4 us against 29.6 us for the two calls).  Only that kernel's
 * one-band form takes them: ttmi_matmul_bfp_ab_supported() says (1 / 0) whether a shape goes there (m == 32 per batch
 * slice: decode); for other shapes, and for BFLOAT4_B activations, the call returns TTMI_ERR_UNSUPPORTED and the caller
 * expands A first (one pass over A, as the GEMMs for tall shapes expand the weights in a pass of their own).
 * Workspace: ttmi_matmul_bfp_workspace_bytes(). */
TTMI_API int ttmi_matmul_bfp_ab_supported(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int a_fmt, int b_fmt);
TTMI_API int ttmi_matmul_bfp_ab(const uint32_t *a, int a_fmt, const uint32_t *b, int b_fmt, uint32_t batch, uint32_t b_batch, uint32_t m,
                       uint32_t k, uint32_t n, const void *bias, int activation, void *c, int c_layout, int c_dtype, void *workspace,
                       size_t workspace_bytes, void *stream);

/* Which kernel a block-float GEMM of this shape and these dtypes goes to, for whoever reads a profiler trace (no counterpart
 * in the reference, whose program factories log their choice; needs no GPU):
 *   out[0]  1 = 64-column streaming kernel, 2 = 128-column streaming kernel, 3 = fused tiled kernels, 4 = expansion + bf16 GEMM
 *   out[1]  k ranges per output (workgroups that share an output), streaming kernels only, else 0
 *   out[2]  workgroups launched where the library knows nothing about workgroup placement
 *   out[3]  workgroups launched on a device whose consecutive workgroups go to 8 XCDs in turn (MI355X) */
TTMI_API void ttmi_matmul_bfp_plan(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int a_dtype, int b_fmt, int c_dtype, uint32_t out[4]);

/* ttnn.matmul / tt_lib.tensor.matmul / bmm with two bf16 operands (ttnn/cpp/ttnn/operations/matmul.hpp:39-42,
 * tt_eager/tt_dnn/op_library/bmm/bmm_op.hpp:388-456):  C[b, m, n] = act(A[b, m, k] . B[(b | 0), k, n] + bias[n]).
 *   b        bf16 in TILE layout (4-face tiles of 2048 bytes, tile (kt, nt) of slice s at index (s*Kt + kt)*Nt + nt), k and n
 *            multiples of 32
 * Everything else as for ttmi_matmul_bfp.  Two launches: the weights are re-laid-out into the operand layout of the matrix
 * cores (workspace: 2 bytes per weight, ttmi_matmul_bf16_workspace_bytes(); NULL = a buffer of the library), then the
 * bf16 GEMM that ttmi_matmul_bfp uses from 512 rows on runs on them.  Not a tuned path: block-float weights are. */
TTMI_API size_t ttmi_matmul_bf16_workspace_bytes(uint32_t b_batch, uint32_t k, uint32_t n);
TTMI_API int ttmi_matmul_bf16(const void *a, int a_layout, const void *b, uint32_t batch, uint32_t b_batch, uint32_t m, uint32_t k,
                     uint32_t n, const void *bias, int activation, void *c, int c_layout, int c_dtype, void *workspace,
                     size_t workspace_bytes, void *stream);

/* A gated pair of GEMMs in one launch:  C[b, m, n] = act(A . B_gate + bias) * (A . B_up), what a gated MLP issues as
 * ttnn.linear(x, w1, activation="silu"), ttnn.linear(x, w3) and ttnn.mul (models/demos/mistral7b/tt/mistral_mlp.py:43-82:
 * three device ops and two [m, n] intermediates there).  Both weight tensors have the shape, format and layout that
 * ttmi_matmul_bfp takes for b; the other arguments mean what they mean there.  The two GEMMs share their activation loads,
 * their launch and the hand-over of partial sums.  Meant for decode shapes (the weights are streamed once per 32 rows of A).
 * The workspace, when the caller brings one, has ttmi_matmul_bfp_gated_workspace_bytes() bytes. */
TTMI_API size_t ttmi_matmul_bfp_gated_workspace_bytes(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt);
TTMI_API int ttmi_matmul_bfp_gated(const void *a, int a_layout, const uint32_t *b_gate, const uint32_t *b_up, int b_fmt, uint32_t batch,
                          uint32_t b_batch, uint32_t m, uint32_t k, uint32_t n, const void *bias, int activation, void *c,
                          int c_layout, int c_dtype, void *workspace, size_t workspace_bytes, void *stream);

/* ttmi_matmul_bfp for callers that cannot allocate device memory: code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and results as
 * ttmi_matmul_bfp without the workspace pair; the scratch of the kernels lies in a static device array of
 * TTMI_STATIC_SCRATCH_BYTES (16 MiB) that every GPU the library runs on holds until the process ends, so the call
 * allocates nothing (no hipMalloc, hipFree or hipHostMalloc; the first call on a device resolves the array's address,
 * which is when the runtime places the array).  Shapes whose scratch does not fit
 * (ttmi_matmul_bfp_workspace_bytes() > TTMI_STATIC_SCRATCH_BYTES: in practice GEMMs of 512 rows and more, whose weights
 * are expanded to 2 bytes each) are rejected with TTMI_ERR_UNSUPPORTED; every output dtype that ttmi_matmul_bfp takes
 * is served.  All calls on one GPU share the one array: calls
 * that overlap in time on one GPU (two streams, two host threads) race and give wrong results — keep them on one
 * stream.  A wait that gives up is reported through ttmi_device_status() only if the device's error word already exists
 * (call ttmi_device_status() once beforehand, where allocating is allowed). */
#define TTMI_STATIC_SCRATCH_BYTES (16u << 20)
TTMI_API int ttmi_matmul_bfp_static(const void *a, int a_layout, const uint32_t *b, int b_fmt, uint32_t batch, uint32_t b_batch,
                           uint32_t m, uint32_t k, uint32_t n, const void *bias, int activation, void *c, int c_layout,
                           int c_dtype, void *stream);

/* c[i] = op(a[i], b[i]) on bf16 tensors of equal shape and layout (count elements, any layout: equal shapes have equal
 * element order), fp32 arithmetic, one rounding to bf16: tt::tt_metal::eltwise_binary
 * (tt_eager/tt_dnn/op_library/eltwise_binary/eltwise_binary_op.hpp:108-140) as reached from ttnn.mul / add / sub
 * (ttnn/ttnn/operations/binary.py:321-424; Mistral's MLP multiplies gate and up projections with it,
 * models/demos/mistral7b/tt/mistral_mlp.py:66-70).  b == NULL: op(a[i], scalar), the *_unary forms
 * (binary.py:360-368).  Unary ops (TTMI_OP_RELU | GELU | SILU, eltwise_unary_op.hpp:17-90) ignore b and scalar.
 * a, b, c 16-byte aligned; c may alias a or b. */
TTMI_API int ttmi_eltwise_bf16(int op, const void *a, const void *b, float scalar, void *c, size_t count, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TTMI_H */
