// Internal declarations shared by the HIP translation units of libttmi.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "ttmi.h"

namespace ttmi {

// Records a message for ttmi_last_error() on this thread and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// hipGetLastError() after a launch -> status.
int check_launch(const char *what);
int check_hip(hipError_t e, const char *what);

// ---- host state (host_state.hip) --------------------------------------------------------------------------------------
enum { SCRATCH_SLOTS = 0, SCRATCH_EXPANDED = 1, SCRATCH_KINDS = 2 };
// The library's own device buffer of at least `bytes` for this purpose on the current device and this stream.  *fresh is
// set when the contents are undefined (a new buffer, or one invalidated since): the caller initialises ALL of it on `stream`
// (*capacity bytes: buffers grow geometrically, so a later, larger request may be served without being fresh).
int scratch_get(int kind, hipStream_t stream, size_t bytes, void **ptr, bool *fresh, size_t *capacity = nullptr);
void scratch_invalidate(int kind);
uint64_t scratch_generation(int kind);      // raised by scratch_invalidate
size_t scratch_grown_size(size_t have, size_t need);
// Device and host address of the current device's error word (either may be null).
int error_word(uint32_t **device_ptr, volatile uint32_t **host_ptr);
bool error_word_if_exists(uint32_t **device_ptr, volatile uint32_t **host_ptr);     // never allocates
// Knobs of the test entry point ttmi_test_set_knob(which, value, set), which only the test build of the library has
// (-DTTMI_TEST_HOOKS: libttmi_test.so); in the product library every knob reads as unset.
enum {
    TTMI_KNOB_MATMUL_KERNEL = 0,      // 1 stream (64 columns), 2 wide (128 columns), 3 tiled, 4 expanded
    TTMI_KNOB_MATMUL_WORKGROUPS = 1,  // workgroups the streaming kernels aim for
    TTMI_KNOB_MATMUL_BLOCK = 2,       // block form of the tiled kernels: 256, 128 (eight wavefronts), 4 (128 rows, four wavefronts), 384
    TTMI_KNOB_SPIN_LIMIT = 3,         // polls before a bounded wait gives up
    TTMI_KNOB_DROP_PARTIAL_SUMS = 4,  // producers do not publish their partial sums (so that a wait must give up)
    TTMI_KNOB_XCDS = 5,               // 1: the 128-column kernel assumes nothing about where workgroups run (device-scope hand-over)
    TTMI_KNOB_COUNT = 6
};
#ifdef TTMI_TEST_HOOKS
bool knob(int which, uint32_t *value);
uint32_t knob_or(int which, uint32_t fallback);
#else
// the product library has no knobs and no test entry points: they exist in libttmi_test.so only (build.py)
inline bool knob(int, uint32_t *) { return false; }
inline uint32_t knob_or(int, uint32_t fallback) { return fallback; }
#endif

int codec_pack_chunks(int fmt, const float *src, size_t n_tiles, int row_major_input, uint32_t *dst, hipStream_t st);
int codec_unpack_chunks(int fmt, const uint32_t *words, size_t n_tiles, int row_major_output, float *dst, hipStream_t st);
int codec_pack_tensor(int fmt, const void *src, int elem, uint32_t batch, uint32_t h, uint32_t w, size_t row_stride,
                      size_t batch_stride, uint32_t *dst, hipStream_t st);
int codec_unpack_tensor(int fmt, const uint32_t *words, uint32_t batch, uint32_t h, uint32_t w, void *dst, int elem,
                        hipStream_t st);
int codec_relayout(bool to_tiles, const void *src, uint32_t elem, uint32_t batch, uint32_t h, uint32_t w, void *dst,
                   hipStream_t st);

int codec_copy_window(int dtype, const void *src, const uint32_t src_shape[4], void *dst, const uint32_t dst_shape[4],
                      const int32_t offset[4], float fill, hipStream_t st);

int codec_typecast_tiles(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n_tiles, hipStream_t st);
int codec_unpad_tiles(uint32_t tile_bytes, const void *src, const uint32_t src_tiles[4], void *dst, const uint32_t start[4],
                      const uint32_t dst_tiles[4], hipStream_t st);

int eltwise_bf16(int op, const void *a, const void *b, float scalar, void *c, size_t count, hipStream_t st);

struct MatmulArgs {
    const void *a; int a_layout;
    const uint32_t *b; int b_fmt;
    uint32_t batch, b_batch, m, k, n;
    const void *bias; int activation;
    void *c; int c_layout, c_dtype;
    void *workspace; size_t workspace_bytes;
    const uint32_t *b2 = nullptr;   // gated form (128-column kernel only): c = act(a . b) * (a . b2)
    size_t workspace_empty_bytes = 0;            // this many leading bytes of the workspace are known to hold nothing but empty slots
    size_t *workspace_left_empty_bytes = nullptr;   // out: as above, after a launch that keeps its partial sums there (untouched otherwise)
    int a_dtype = TTMI_BFLOAT16;    // TTMI_BFLOAT8_B: `a` holds packed tiles (TILE layout), which the 128-column kernel expands itself
    bool no_alloc = false;          // the call may not allocate: `workspace` is all the scratch there is, its last 256 bytes stand
                                    // in for the error word when the device has none yet
};
// the argument checks of the matmul entry points (everything but the workspace); dense bf16 weights pass only where the
// caller says so (ttmi_matmul_bf16): every other entry point decodes `b` as packed block-float tiles
int validate_matmul(const void *a, int a_layout, const uint32_t *b, int b_fmt, uint32_t batch, uint32_t b_batch, uint32_t m, uint32_t k,
                    uint32_t n, int activation, const void *c, int c_layout, int c_dtype, bool allow_bf16_weights = false);
size_t matmul_workspace_bytes(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt);
int matmul_bfp(const MatmulArgs &args, hipStream_t st);         // streaming kernel (decode shapes) or the tiled one
void matmul_plan(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt, bool a_or_c_bfp, uint32_t out[4]);
bool matmul_takes_bfp_activations(uint32_t batch, uint32_t m, uint32_t k, uint32_t n, int b_fmt);   // args.a_dtype = TTMI_BFLOAT8_B goes through for this shape
int matmul_bfp_stream(const MatmulArgs &args, hipStream_t st);
int matmul_bfp_wide(const MatmulArgs &args, hipStream_t st);     // the streaming kernel with 128-column units
size_t matmul_gated_workspace_bytes(uint32_t batch, uint32_t m, uint32_t k, uint32_t n);
int matmul_bfp_gated(const MatmulArgs &args, hipStream_t st);   // args.b2 set
int matmul_bf16(const MatmulArgs &args, hipStream_t st);        // args.b: bf16 tiles, args.b_fmt = TTMI_BFLOAT16
int matmul_bfp_tiled(const MatmulArgs &args, hipStream_t st);
int matmul_bfp_expanded(const MatmulArgs &args, hipStream_t st);   // expand the weights to bf16 once, then a bf16 GEMM
size_t matmul_expanded_workspace_bytes(uint32_t b_batch, uint32_t k, uint32_t n);

}  // namespace ttmi
