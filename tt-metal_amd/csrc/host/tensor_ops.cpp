// Host side of the TT-NN / tt_lib surface for block-float tensors (see tensor_ops.hpp).  Every conversion and every GEMM
// is a call into the C ABI of include/ttmi.h; this file decides which calls, in which order, on which shapes, and says no
// where the reference says no.
#include "tensor_ops.hpp"

#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstring>
#include <stdexcept>

#include "ttmi.h"

namespace ttmi::host {

namespace {

Runtime g_runtime;

[[noreturn]] void raise(const std::string &message) { throw std::runtime_error(message); }

void check(int status) {
    if (status != TTMI_OK) raise(ttmi_last_error());
}
void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) raise(std::string(what) + ": " + hipGetErrorString(e));
}

void need_gpu() {
    if (!g_runtime.allocate || !g_runtime.gpu_available || !g_runtime.gpu_available())
        raise("no GPU visible: block-float conversions and matmuls run as HIP kernels and have no CPU fallback");
}

struct DeviceGuard {
    int previous = 0;
    bool switched = false;
    explicit DeviceGuard(int device) {
        hip_check(hipGetDevice(&previous), "hipGetDevice");
        if (device >= 0 && device != previous) { hip_check(hipSetDevice(device), "hipSetDevice"); switched = true; }
    }
    ~DeviceGuard() { if (switched) (void)hipSetDevice(previous); }
};

int current_device() {
    int d = 0;
    hip_check(hipGetDevice(&d), "hipGetDevice");
    return d;
}

void *stream_of(int device) { return g_runtime.stream ? g_runtime.stream(device) : nullptr; }

Buffer allocate(size_t nbytes, int device) {
    if (!g_runtime.allocate) raise("ttmi host layer: no runtime set (memory comes from the embedding)");
    Buffer b = g_runtime.allocate(nbytes ? nbytes : 1, device);
    b.nbytes = nbytes;
    b.device = device;
    return b;
}

// copies between host and device memory on the runtime's stream and waits for it
void copy(Buffer &dst, const Buffer &src, size_t nbytes) {
    if (!nbytes) return;
    if (dst.device < 0 && src.device < 0) { std::memcpy(dst.data, src.data, nbytes); return; }
    const int device = dst.device >= 0 ? dst.device : src.device;
    DeviceGuard guard(device);
    hipStream_t st = (hipStream_t)stream_of(device);
    const hipMemcpyKind kind = dst.device < 0 ? hipMemcpyDeviceToHost : src.device < 0 ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice;
    hip_check(hipMemcpyAsync(dst.data, src.data, nbytes, kind, st), "hipMemcpyAsync");
    hip_check(hipStreamSynchronize(st), "hipStreamSynchronize");
    // Data that leaves the device is where a user first looks at a result: whatever a kernel has reported by now (a bounded
    // wait that gave up) is raised here, not at the next launch.
    if (kind == hipMemcpyDeviceToHost) check(ttmi_device_status());
}

Buffer moved_to(const Buffer &src, int device) {
    if (src.device == device) return src;
    Buffer dst = allocate(src.nbytes, device);
    copy(dst, src, src.nbytes);
    return dst;
}

uint64_t product(const Dims &d, size_t from = 0, size_t to = (size_t)-1) {
    uint64_t v = 1;
    for (size_t i = from; i < d.size() && i < to; ++i) v *= d[i];
    return v;
}

uint32_t pad32(uint32_t x) { return (x + 31u) / 32u * 32u; }

struct BatchHW { uint32_t batch, h, w; };
BatchHW batch_h_w(const Dims &shape) {
    if (shape.size() > 4) raise("Rank " + std::to_string(shape.size()) + " is not supported!");     // tensor_impl.hpp:143-155
    if (shape.empty()) return {1, 1, 1};
    const uint32_t w = shape.back(), h = shape.size() > 1 ? shape[shape.size() - 2] : 1;
    return {(uint32_t)product(shape, 0, shape.size() > 2 ? shape.size() - 2 : 0), h, w};
}

std::string list_of(const Dims &d) {
    std::string s = "[";
    for (size_t i = 0; i < d.size(); ++i) s += (i ? ", " : "") + std::to_string(d[i]);
    return s + "]";
}

Dims as4(const Dims &d) {
    Dims out(4 - d.size(), 1);
    out.insert(out.end(), d.begin(), d.end());
    return out;
}

Tensor like(const Tensor &t, Buffer buffer) {
    Tensor out = t;
    out.buffer = std::move(buffer);
    return out;
}

// Runs `work(device buffer of t) -> device buffer` and brings the result to where t lives: host tensors are staged through
// the current GPU (the reference does these steps on the CPU; here every one of them is a kernel).
template <typename Work> Buffer through_gpu(const Tensor &t, Work work) {
    need_gpu();
    const int device = t.on_device() ? t.buffer.device : current_device();
    DeviceGuard guard(device);
    Buffer result = work(moved_to(t.buffer, device), device);
    return t.on_device() ? result : moved_to(result, -1);
}

size_t words_bytes(DataType dtype, uint64_t elements) { return (size_t)(elements / 1024 * ttmi_tile_size((int)dtype)); }

// ---- kernels behind the C ABI, on device buffers ----------------------------------------------------------------------------
Buffer pack_chunks(DataType fmt, const Buffer &fp32, uint64_t elements, int device) {
    Buffer out = allocate(words_bytes(fmt, elements), device);
    check(ttmi_pack_fp32_vec_as_bfp_tiles((int)fmt, (const float *)fp32.data, elements / 1024, 0, (uint32_t *)out.data, stream_of(device)));
    return out;
}
Buffer unpack_chunks(DataType fmt, const Buffer &words, uint64_t elements, int device) {
    Buffer out = allocate(elements * 4, device);
    check(ttmi_unpack_bfp_tiles_into_float_vec((int)fmt, (const uint32_t *)words.data, elements / 1024, 0, (float *)out.data, stream_of(device)));
    return out;
}
Buffer relayout(bool to_tiles, const Buffer &src, size_t elem, const BatchHW &s, int device) {
    const uint64_t out_elements = to_tiles ? (uint64_t)s.batch * pad32(s.h) * pad32(s.w) : (uint64_t)s.batch * s.h * s.w;
    Buffer out = allocate(out_elements * elem, device);
    if (to_tiles) check(ttmi_tilize(src.data, (uint32_t)elem, s.batch, s.h, s.w, out.data, stream_of(device)));
    else check(ttmi_untilize(src.data, (uint32_t)elem, s.batch, s.h, s.w, out.data, stream_of(device)));
    return out;
}
Buffer typecast_tiles(const Buffer &src, DataType from, DataType to, uint64_t elements, int device) {
    const size_t bytes = is_block_float(to) ? words_bytes(to, elements) : elements * element_bytes(to);
    Buffer out = allocate(bytes, device);
    check(ttmi_typecast_tiles(src.data, (int)from, out.data, (int)to, elements / 1024, stream_of(device)));
    return out;
}
Buffer window(DataType dtype, const Buffer &src, const Dims &src_shape, const Dims &dst_shape, const int32_t offset[4], float fill, int device) {
    const uint64_t volume = product(dst_shape);
    const size_t bytes = is_block_float(dtype) ? words_bytes(dtype, volume) : volume * element_bytes(dtype);
    Buffer out = allocate(bytes, device);
    check(ttmi_copy_window((int)dtype, src.data, src_shape.data(), out.data, dst_shape.data(), offset, fill, stream_of(device)));
    return out;
}

// Kernels index a buffer by the tensor's shape: a tensor whose buffer does not hold exactly what its shape, dtype and layout
// say (a truncated or stale cache file, a raw buffer of the wrong size) is refused before any of them can run.
void check_consistent(const Tensor &t, const std::string &what) {
    if (!element_bytes(t.dtype) && !is_block_float(t.dtype)) raise(what + ": unsupported DataType " + std::to_string((int)t.dtype));
    if (t.layout != Layout::ROW_MAJOR && t.layout != Layout::TILE) raise(what + ": unsupported Layout " + std::to_string((int)t.layout));
    for (size_t i = 0; i < t.shape.size(); ++i)
        if (t.shape[i] > t.padded[i]) raise(what + ": dimension " + std::to_string(i) + " is larger without padding (" + std::to_string(t.shape[i]) + ") than with it (" + std::to_string(t.padded[i]) + ")");
    const uint64_t volume = product(t.padded);
    if (is_block_float(t.dtype) && volume % 1024) raise(what + ": a block-float tensor holds whole tiles, " + std::to_string(volume) + " elements are not");
    if (t.layout == Layout::TILE && !t.padded.empty()) {
        const size_t r = t.padded.size();
        if (t.padded[r - 1] % 32 || (r > 1 && t.padded[r - 2] % 32)) raise(what + ": the last two dimensions of a TILE tensor must be multiples of 32");
    }
    const size_t expected = storage_bytes(t.dtype, t.layout, t.padded);
    if (t.buffer.nbytes != expected)
        raise(what + ": the buffer holds " + std::to_string(t.buffer.nbytes) + " bytes, shape " + list_of(t.padded) + " of " + name_of(t.dtype) + " needs " + std::to_string(expected));
}

void require_rank4(const Dims &d, const char *what) {
    if (d.size() != 4) raise(std::string(what) + ": shapes must have rank 4");
}

}  // namespace

void set_runtime(Runtime runtime) { g_runtime = std::move(runtime); }

uint64_t Tensor::volume() const { return product(padded); }
bool is_block_float(DataType dtype) { return dtype == DataType::BFLOAT8_B || dtype == DataType::BFLOAT4_B; }
size_t element_bytes(DataType dtype) {
    switch (dtype) {
        case DataType::BFLOAT16: case DataType::UINT16: return 2;
        case DataType::FLOAT32: case DataType::UINT32: return 4;
        default: return 0;
    }
}
size_t storage_bytes(DataType dtype, Layout, const Dims &padded) {
    const uint64_t v = product(padded);
    return is_block_float(dtype) ? words_bytes(dtype, v) : (size_t)(v * element_bytes(dtype));
}
const char *name_of(DataType dtype) {
    switch (dtype) {
        case DataType::BFLOAT16: return "BFLOAT16";
        case DataType::FLOAT32: return "FLOAT32";
        case DataType::UINT32: return "UINT32";
        case DataType::BFLOAT8_B: return "BFLOAT8_B";
        case DataType::BFLOAT4_B: return "BFLOAT4_B";
        case DataType::UINT16: return "UINT16";
        default: return "INVALID";
    }
}
const char *name_of(Layout layout) { return layout == Layout::ROW_MAJOR ? "ROW_MAJOR" : layout == Layout::TILE ? "TILE" : "INVALID"; }

// ---------------------------------------------------------------------------------------------------------------------------
// tt_lib.tensor.Tensor
// ---------------------------------------------------------------------------------------------------------------------------
Tensor from_host(const void *data, const Dims &shape, DataType dtype) {
    Tensor t;
    t.shape = t.padded = shape;
    t.dtype = dtype;
    t.layout = Layout::ROW_MAJOR;
    const uint64_t volume = product(shape);
    if (is_block_float(dtype)) {
        // pytensor.cpp:78-85,145-157: the fp32 values are packed in consecutive 1024-element chunks and the tensor is declared ROW_MAJOR
        if (volume % 1024) raise("TT_ASSERT: fp32_vec.size() % num_float_in_tile == 0 (block-float tensors hold whole tiles)");
        need_gpu();
        const int device = current_device();
        Buffer host{const_cast<void *>(data), (size_t)volume * 4, -1, nullptr};
        Buffer staged = moved_to(host, device);
        t.buffer = moved_to(pack_chunks(dtype, staged, volume, device), -1);
        return t;
    }
    const size_t bytes = (size_t)volume * element_bytes(dtype);
    if (!element_bytes(dtype)) raise(std::string("Unsupported DataType: ") + name_of(dtype));
    t.buffer = allocate(bytes, -1);
    if (bytes) std::memcpy(t.buffer.data, data, bytes);
    return t;
}

Tensor wrap(Buffer buffer, const Dims &shape, const Dims &padded, DataType dtype, Layout layout) {
    if (shape.size() != padded.size()) raise("Shape: rank of the shape and of the shape with tile padding differ");
    Tensor t;
    t.buffer = std::move(buffer);
    t.shape = shape; t.padded = padded; t.dtype = dtype; t.layout = layout;
    check_consistent(t, "Tensor");
    return t;
}

Tensor to_layout(const Tensor &t, Layout target) {
    if (target == t.layout) return t;
    const BatchHW s = batch_h_w(t.padded);
    const uint64_t volume = t.volume();
    Tensor out = t;
    out.layout = target;
    if (target == Layout::TILE) {
        if (s.w % 32 || (t.padded.size() > 1 && s.h % 32))
            raise("TT_ASSERT: Unsupported shape for tensor conversion (height and width must be multiples of 32)");
        out.buffer = through_gpu(t, [&](const Buffer &src, int device) {
            if (is_block_float(t.dtype))   // tensor_impl.cpp:179-197: unpack -> tilize as fp32 -> pack
                return pack_chunks(t.dtype, relayout(true, unpack_chunks(t.dtype, src, volume, device), 4, s, device), volume, device);
            return relayout(true, src, element_bytes(t.dtype), s, device);
        });
        return out;
    }
    out.buffer = through_gpu(t, [&](const Buffer &src, int device) {
        if (is_block_float(t.dtype))
            return pack_chunks(t.dtype, relayout(false, unpack_chunks(t.dtype, src, volume, device), 4, s, device), volume, device);
        return relayout(false, src, element_bytes(t.dtype), s, device);
    });
    return out;
}

Tensor to_device(const Tensor &t, int device) {
    need_gpu();
    return like(t, moved_to(t.buffer, device));
}
Tensor to_host(const Tensor &t) { return like(t, moved_to(t.buffer, -1)); }

Tensor reshape(const Tensor &t, const Dims &logical, const Dims &padded) {
    if (logical.size() != padded.size()) raise("Shape: rank of the shape and of the shape with tile padding differ");
    if (product(padded) != t.volume())
        raise("TT_ASSERT: reshape changes the volume (" + std::to_string(t.volume()) + " -> " + std::to_string(product(padded)) + ")");
    if (t.layout == Layout::TILE) {
        const size_t r0 = t.padded.size(), r1 = padded.size();
        const bool same = r0 >= 2 && r1 >= 2 && t.padded[r0 - 1] == padded[r1 - 1] && t.padded[r0 - 2] == padded[r1 - 2];
        if (!same) raise("reshape of a TILE tensor must keep the last two padded dimensions");
    }
    Tensor out = t;
    out.shape = logical; out.padded = padded;
    return out;
}

Tensor to_torch(const Tensor &t) {
    if (t.on_device()) raise("Tensor must be on host to be converted to torch (call .cpu() first)");
    if (is_block_float(t.dtype)) {       // pytensor.cpp:382-393: sequential unpack, fp32
        Tensor out = t;
        out.dtype = DataType::FLOAT32;
        const uint64_t volume = t.volume();
        out.buffer = through_gpu(t, [&](const Buffer &src, int device) { return unpack_chunks(t.dtype, src, volume, device); });
        return out;
    }
    Tensor out = t;
    out.buffer = allocate(t.buffer.nbytes, -1);
    copy(out.buffer, t.buffer, t.buffer.nbytes);
    return out;
}

// ---- pad / unpad on the host (tensor.cpp:204-260, tensor_impl.hpp:508-660, tensor_impl.cpp:200-283) ---------------------------
namespace {
Tensor host_window(const Tensor &t, const Dims &dst_shape, const int32_t offset[4], float fill, const char *what) {
    if (t.on_device()) raise("TT_THROW: Device storage isn't supported");                    // tensor_impl.hpp:590, 675
    if (t.layout != Layout::ROW_MAJOR) raise(std::string("TT_ASSERT: Tensor layout must be ROW_MAJOR for ") + what);
    require_rank4(t.padded, what);
    require_rank4(dst_shape, what);
    if (is_block_float(t.dtype) && product(dst_shape) % 1024)
        raise("TT_ASSERT: fp32_vec.size() % num_float_in_tile == 0 (block-float tensors hold whole tiles)");
    Tensor out = t;
    out.buffer = through_gpu(t, [&](const Buffer &src, int device) { return window(t.dtype, src, t.padded, dst_shape, offset, fill, device); });
    return out;
}
}  // namespace

Tensor pad(const Tensor &t, const Dims &output_shape, const Dims &input_start, float pad_value) {
    require_rank4(output_shape, "pad"); require_rank4(input_start, "pad"); require_rank4(t.padded, "pad");
    int32_t offset[4];
    for (int i = 0; i < 4; ++i) {
        if ((uint64_t)t.padded[i] + input_start[i] > output_shape[i])                            // tensor_impl.hpp:522-525
            raise("TT_ASSERT: input_tensor_shape[" + std::to_string(i) + "] + input_tensor_start[" + std::to_string(i) + "] <= output_tensor_shape[" +
                  std::to_string(i) + "]");
        offset[i] = (int32_t)input_start[i];
    }
    Tensor out = host_window(t, output_shape, offset, pad_value, "padding");
    out.shape = t.padded;
    out.padded = output_shape;
    return out;
}

Tensor unpad(const Tensor &t, const Dims &start, const Dims &end) {
    require_rank4(start, "unpad"); require_rank4(end, "unpad"); require_rank4(t.padded, "unpad");
    int32_t offset[4];
    Dims out_shape(4);
    for (int i = 0; i < 4; ++i) {                                                               // tensor_impl.hpp:614-627
        if (start[i] >= t.padded[i] || end[i] >= t.padded[i] || start[i] > end[i])
            raise("TT_ASSERT: output_tensor_start[" + std::to_string(i) + "] <= output_tensor_end[" + std::to_string(i) + "] < input_tensor_shape[" +
                  std::to_string(i) + "]");
        offset[i] = -(int32_t)start[i];
        out_shape[i] = end[i] - start[i] + 1;
    }
    Tensor out = host_window(t, out_shape, offset, 0.f, "unpadding");
    out.shape = out.padded = out_shape;
    return out;
}

Tensor pad_to_tile(const Tensor &t, float pad_value) {
    require_rank4(t.padded, "pad_to_tile");
    return pad(t, {t.padded[0], t.padded[1], pad32(t.padded[2]), pad32(t.padded[3])}, {0, 0, 0, 0}, pad_value);
}

Tensor unpad_from_tile(const Tensor &t, const Dims &out) {
    require_rank4(out, "unpad_from_tile"); require_rank4(t.padded, "unpad_from_tile");
    if (t.padded[0] != out[0] || t.padded[1] != out[1]) raise("TT_ASSERT: Input shape must match output shape apart from last 2 dims");
    if (t.padded[2] % 32 || t.padded[3] % 32) raise("TT_ASSERT: Last 2 dims of input shape must be multiples of 32");
    if (!(t.padded[2] < out[2] + 32 && out[2] <= t.padded[2] && t.padded[3] < out[3] + 32 && out[3] <= t.padded[3]) || !out[2] || !out[3])
        raise("TT_ASSERT: Last 2 dims of output must be within range to have been padded to input");
    return unpad(t, {0, 0, 0, 0}, {out[0] - 1, out[1] - 1, out[2] - 1, out[3] - 1});
}

Tensor device_unpad(const Tensor &t, const Dims &start, const Dims &end) {
    if (!t.on_device()) raise("TT_FATAL: Operands to unpad need to be on device!");
    require_rank4(start, "unpad"); require_rank4(end, "unpad"); require_rank4(t.padded, "unpad");
    Dims out_shape(4);
    for (int i = 0; i < 4; ++i) {
        if (start[i] >= t.padded[i] || end[i] >= t.padded[i] || start[i] > end[i])
            raise("TT_FATAL: output_tensor_start[" + std::to_string(i) + "] <= output_tensor_end[" + std::to_string(i) + "] < input shape[" + std::to_string(i) + "]");
        out_shape[i] = end[i] - start[i] + 1;
    }
    const int device = t.buffer.device;
    DeviceGuard guard(device);
    Tensor out = t;
    out.shape = out.padded = out_shape;
    if (t.layout == Layout::TILE) {
        if (out_shape[2] % 32 || start[2] % 32 || out_shape[3] % 32 || start[3] % 32) raise("TT_FATAL: Can only unpad tilized tensor with full tiles");
        const uint32_t src_tiles[4] = {t.padded[0], t.padded[1], t.padded[2] / 32, t.padded[3] / 32};
        const uint32_t at[4] = {start[0], start[1], start[2] / 32, start[3] / 32};
        const uint32_t dst_tiles[4] = {out_shape[0], out_shape[1], out_shape[2] / 32, out_shape[3] / 32};
        out.buffer = allocate((size_t)product(out_shape) / 1024 * ttmi_tile_size((int)t.dtype), device);
        check(ttmi_unpad_tiles((int)t.dtype, t.buffer.data, src_tiles, out.buffer.data, at, dst_tiles, stream_of(device)));
        return out;
    }
    if (is_block_float(t.dtype)) raise("TT_FATAL: block-float tensors on device are in TILE layout");
    const size_t elem = element_bytes(t.dtype);
    if ((out_shape[3] * elem) % 4 || (start[3] * elem) % 4) raise("TT_FATAL: RM unpadding requires output X size to be packable");
    const int32_t offset[4] = {-(int32_t)start[0], -(int32_t)start[1], -(int32_t)start[2], -(int32_t)start[3]};
    out.buffer = window(t.dtype, t.buffer, t.padded, out_shape, offset, 0.f, device);
    return out;
}

// ---------------------------------------------------------------------------------------------------------------------------
// matmul
// ---------------------------------------------------------------------------------------------------------------------------
Tensor matmul(const Tensor &a, const Tensor &b, bool bcast_batch, const Tensor *bias, int activation, std::optional<DataType> output_dtype,
              const std::string &op, bool untilize_out) {
    const std::pair<const Tensor *, const char *> operands[2] = {{&a, "input_tensor_a"}, {&b, "input_tensor_b"}};
    for (const auto &[t, name] : operands) {
        if (!t->on_device()) raise("TT_FATAL: Operands to " + op + " need to be on device! (" + name + ")");
        if (t->layout != Layout::TILE) raise("TT_FATAL: Inputs to " + op + " must be tilized (" + name + ")");
    }
    const Dims &pa = a.padded, &pb = b.padded;
    if (pa.size() < 2 || pb.size() < 2 || pa.size() > 4 || pb.size() > 4) raise("TT_FATAL: " + op + " supports ranks 2 to 4");
    if (pa.back() != pb[pb.size() - 2])
        raise("TT_FATAL: The width of the first tensor must be equal to the height of the second tensor (a.shape[-1] = " + std::to_string(pa.back()) +
              ", b.shape[-2] = " + std::to_string(pb[pb.size() - 2]) + ")");
    if (!is_block_float(b.dtype) && b.dtype != DataType::BFLOAT16)
        raise(std::string("TT_FATAL: Unsupported data format for input b: ") + name_of(b.dtype));               // bmm_op.cpp:839
    if (a.dtype != DataType::BFLOAT16 && !is_block_float(a.dtype))
        raise(std::string("TT_FATAL: Unsupported data format for input a: ") + name_of(a.dtype));      // bmm_op.cpp:839
    const uint32_t batch_a = (uint32_t)product(pa, 0, pa.size() - 2), batch_b = (uint32_t)product(pb, 0, pb.size() - 2);
    if (bcast_batch) {
        if (batch_b != 1) raise("TT_FATAL: matmul (batch bcast variant) expects input tensors of shapes BCMK*11KN=BCMN");   // bmm_op.cpp:529
    } else if (batch_b != batch_a) {
        raise("TT_FATAL: bmm (non-bcast matmul) expects input tensors of shapes BCMK*BCKN=BCMN");                         // bmm_op.cpp:533
    }
    const uint32_t m = pa[pa.size() - 2], k = pa.back(), n = pb.back();
    const DataType out_dtype = output_dtype ? *output_dtype : a.dtype;      // bmm_op.hpp:388: the output takes input a's dtype
    if (out_dtype != DataType::BFLOAT16 && !is_block_float(out_dtype))
        raise(op + ": output dtype " + name_of(out_dtype) + " is not supported (BFLOAT16, BFLOAT8_B, BFLOAT4_B)");
    if (untilize_out && out_dtype != DataType::BFLOAT16)                                                // bmm_op.cpp:536-538, 865-867
        raise("TT_FATAL: this->output_dtype == DataType::BFLOAT16 (untilize_out writes a ROW_MAJOR output, which a block-float tensor cannot be)");
    const int device = a.buffer.device;
    DeviceGuard guard(device);
    Buffer bias_row;
    if (bias) {
        if (!bias->on_device()) raise("TT_FATAL: bias must be on device");
        if (bias->padded.empty() || bias->padded.back() != n) raise("TT_FATAL: bias width must match the output width");
        if (bias->dtype != DataType::BFLOAT16 && !is_block_float(bias->dtype))
            raise(std::string("TT_FATAL: Unsupported data format for the bias: ") + name_of(bias->dtype));
        // the bias is a [.., 32, N] tile row in the reference; its first row carries the values (matmul.hpp:117-140).  The GEMM
        // reads n bf16 values: a row-major copy of that row.
        const uint32_t bh = bias->padded.size() > 1 ? bias->padded[bias->padded.size() - 2] : 1;
        if (is_block_float(bias->dtype)) {
            bias_row = allocate((size_t)bh * n * 2, device);
            check(ttmi_unpack_bfp_tiles_as_rowmajor((int)bias->dtype, (const uint32_t *)bias->buffer.data, 1, bh, n, bias_row.data, TTMI_BFLOAT16, stream_of(device)));
        } else if (bias->layout == Layout::TILE) {
            bias_row = relayout(false, bias->buffer, 2, {1, bh, n}, device);
        } else {
            bias_row = bias->buffer;
        }
    }
    const uint64_t a_elements = (uint64_t)batch_a * m * k, c_elements = (uint64_t)batch_a * m * n;
    // block-float activations are expanded (exactly) to bf16 tiles by one kernel in front of the GEMM; a block-float output is
    // packed by the GEMM itself, in its epilogue (the host packers' arithmetic on the bf16-rounded sums: parity with the
    // Tensix packer unpinned)
    // ... unless the shape goes to the kernel that streams the weights, which takes BFLOAT8_B activations as they are
    const bool a_in_kernel = is_block_float(b.dtype) && ttmi_matmul_bfp_ab_supported(batch_a, m, k, n, (int)a.dtype, (int)b.dtype);
    Buffer a_tiles = is_block_float(a.dtype) && !a_in_kernel ? typecast_tiles(a.buffer, a.dtype, DataType::BFLOAT16, a_elements, device) : a.buffer;
    const bool packed_out = is_block_float(out_dtype);
    const int c_layout = untilize_out ? TTMI_ROW_MAJOR : TTMI_TILE;                                     // bmm_op.cpp:1069
    Buffer c = allocate(packed_out ? storage_bytes(out_dtype, Layout::TILE, {batch_a, m, n}) : c_elements * 2, device);
    if (b.dtype == DataType::BFLOAT16)      // two bf16 operands: not the tuned path (the weights are re-laid-out on every call), but the same surface
        check(ttmi_matmul_bf16(a_tiles.data, TTMI_TILE, b.buffer.data, batch_a, batch_b, m, k, n, bias ? bias_row.data : nullptr, activation, c.data,
                               c_layout, packed_out ? (int)out_dtype : TTMI_BFLOAT16, nullptr, 0, stream_of(device)));
    else if (a_in_kernel)
        check(ttmi_matmul_bfp_ab((const uint32_t *)a_tiles.data, (int)a.dtype, (const uint32_t *)b.buffer.data, (int)b.dtype, batch_a, batch_b, m, k, n,
                                 bias ? bias_row.data : nullptr, activation, c.data, c_layout, packed_out ? (int)out_dtype : TTMI_BFLOAT16, nullptr, 0,
                                 stream_of(device)));
    else
        check(ttmi_matmul_bfp(a_tiles.data, TTMI_TILE, (const uint32_t *)b.buffer.data, (int)b.dtype, batch_a, batch_b, m, k, n,
                              bias ? bias_row.data : nullptr, activation, c.data, c_layout, packed_out ? (int)out_dtype : TTMI_BFLOAT16, nullptr, 0,
                              stream_of(device)));
    Tensor out;
    out.buffer = std::move(c);
    out.shape.assign(a.shape.begin(), a.shape.end() - 1);
    out.shape.push_back(b.shape.back());
    out.padded.assign(pa.begin(), pa.end() - 1);
    out.padded.push_back(n);
    out.dtype = out_dtype;
    out.layout = untilize_out ? Layout::ROW_MAJOR : Layout::TILE;     // the padded rows and columns stay part of the row-major output
    return out;
}

// silu(x w1) * (x w3) of a gated MLP (models/demos/mistral7b/tt/mistral_mlp.py:43-82 issues it as linear(activation), linear,
// mul) as ONE launch: both weight matrices stream through the same workgroups and share the activation loads.
Tensor matmul_gated(const Tensor &a, const Tensor &b_gate, const Tensor &b_up, int activation, std::optional<DataType> output_dtype,
                    const std::string &op) {
    const std::pair<const Tensor *, const char *> operands[3] = {{&a, "input_tensor_a"}, {&b_gate, "input_tensor_b"}, {&b_up, "input_tensor_c"}};
    for (const auto &[t, name] : operands) {
        if (!t->on_device()) raise("TT_FATAL: Operands to " + op + " need to be on device! (" + name + ")");
        if (t->layout != Layout::TILE) raise("TT_FATAL: Inputs to " + op + " must be tilized (" + name + ")");
    }
    if (a.dtype != DataType::BFLOAT16) raise(std::string("TT_FATAL: Unsupported data format for input a: ") + name_of(a.dtype));
    if (!is_block_float(b_gate.dtype) || b_up.dtype != b_gate.dtype || b_up.padded != b_gate.padded)
        raise("TT_FATAL: " + op + ": the two weight tensors must be block-float tensors of the same dtype and shape");
    const Dims &pa = a.padded, &pb = b_gate.padded;
    if (pa.size() < 2 || pb.size() < 2 || pa.size() > 4 || pb.size() > 4) raise("TT_FATAL: " + op + " supports ranks 2 to 4");
    if (product(pb, 0, pb.size() - 2) != 1) raise("TT_FATAL: " + op + " expects input tensors of shapes BCMK*11KN=BCMN");
    if (pa.back() != pb[pb.size() - 2])
        raise("TT_FATAL: The width of the first tensor must be equal to the height of the second tensor (a.shape[-1] = " + std::to_string(pa.back()) +
              ", b.shape[-2] = " + std::to_string(pb[pb.size() - 2]) + ")");
    const DataType out_dtype = output_dtype ? *output_dtype : a.dtype;
    if (out_dtype != DataType::BFLOAT16 && !is_block_float(out_dtype))
        raise(op + ": output dtype " + name_of(out_dtype) + " is not supported (BFLOAT16, BFLOAT8_B, BFLOAT4_B)");
    const uint32_t batch = (uint32_t)product(pa, 0, pa.size() - 2), m = pa[pa.size() - 2], k = pa.back(), n = pb.back();
    const int device = a.buffer.device;
    DeviceGuard guard(device);
    const bool packed_out = is_block_float(out_dtype);
    Buffer c = allocate(packed_out ? storage_bytes(out_dtype, Layout::TILE, {batch, m, n}) : (size_t)batch * m * n * 2, device);
    check(ttmi_matmul_bfp_gated(a.buffer.data, TTMI_TILE, (const uint32_t *)b_gate.buffer.data, (const uint32_t *)b_up.buffer.data, (int)b_gate.dtype, batch, 1,
                                m, k, n, nullptr, activation, c.data, TTMI_TILE, (int)out_dtype, nullptr, 0, stream_of(device)));
    Tensor out;
    out.buffer = std::move(c);
    out.shape.assign(a.shape.begin(), a.shape.end() - 1);
    out.shape.push_back(b_gate.shape.back());
    out.padded.assign(pa.begin(), pa.end() - 1);
    out.padded.push_back(n);
    out.dtype = out_dtype;
    out.layout = Layout::TILE;
    return out;
}

int activation_code(const std::optional<std::string> &activation) {       // ttnn/ttnn/operations/matmul.py:59-63
    if (!activation) return TTMI_ACT_NONE;
    if (*activation == "relu") return TTMI_ACT_RELU;
    if (*activation == "gelu") return TTMI_ACT_GELU;
    if (*activation == "silu") return TTMI_ACT_SILU;
    raise(*activation + " is not supported as activation function. Use one of these instead: ['relu', 'gelu', 'silu']");
}

namespace {
void ttnn_validate(const std::string &operation_name, const Tensor &t) {
    // validation.hpp:17-74 through matmul.hpp:39-42: rank 2-4; bf16 | bfp8_b | bfp4_b; TILE; on device
    if (t.shape.size() < 2 || t.shape.size() > 4)
        raise(operation_name + ": Tensor must be of rank (2, 3, 4), but got " + std::to_string(t.shape.size()));
    if (t.dtype != DataType::BFLOAT16 && !is_block_float(t.dtype))
        raise(operation_name + ": Tensor must be of type bfloat16, bfloat8_b or bfloat4_b, but got " + name_of(t.dtype));
    if (t.layout != Layout::TILE) raise(operation_name + ": Tensor must be of layout TILE, but got " + name_of(t.layout));
    if (!t.on_device()) raise(operation_name + ": Tensor must be on device!");
}
}  // namespace

Tensor ttnn_matmul(const std::string &operation_name, const Tensor &a, const Tensor &b, const Tensor *bias,
                   const std::optional<std::string> &activation, std::optional<DataType> dtype) {
    ttnn_validate(operation_name, a);
    ttnn_validate(operation_name, b);
    const int act = activation_code(activation);
    if (a.padded.back() != b.padded[b.padded.size() - 2] || a.shape.back() != b.shape[b.shape.size() - 2])
        raise("The width of the first tensor must be equal to the height of the second tensor");      // matmul.hpp:60-62
    const uint64_t batch_b = product(b.padded, 0, b.padded.size() - 2);
    if (batch_b != 1 && activation) raise("Cannot use activation with batched input b");              // matmul.py:215-216
    if (bias) ttnn_validate(operation_name, *bias);
    return matmul(a, b, batch_b == 1, bias, act, dtype, operation_name, false);
}

// ---------------------------------------------------------------------------------------------------------------------------
// elementwise, dtype changes
// ---------------------------------------------------------------------------------------------------------------------------
Tensor eltwise(int op, const Tensor &a, const Tensor *b, float scalar, const std::string &name) {
    const Tensor *operands[2] = {&a, b};
    for (const Tensor *t : operands) {
        if (!t) continue;
        if (!t->on_device()) raise("TT_FATAL: Operands to eltwise ops need to be on device!");
        if (t->dtype != DataType::BFLOAT16 && !is_block_float(t->dtype))
            raise(std::string("TT_FATAL: Unsupported data format ") + name_of(t->dtype) + " (BFLOAT16, BFLOAT8_B, BFLOAT4_B)");
    }
    if (b) {
        if (a.padded != b->padded)
            raise("TT_FATAL: " + name + ": input shapes must be the same (" + list_of(a.padded) + " vs " + list_of(b->padded) + "); broadcast forms are not part of this build");
        if (a.layout != b->layout) raise("TT_FATAL: " + name + ": inputs must have the same layout");
    }
    const int device = a.buffer.device;
    DeviceGuard guard(device);
    const uint64_t count = a.volume();
    auto as_bf16 = [&](const Tensor &t) { return is_block_float(t.dtype) ? typecast_tiles(t.buffer, t.dtype, DataType::BFLOAT16, count, device) : t.buffer; };
    Buffer x = as_bf16(a), y;
    if (b) y = as_bf16(*b);
    Buffer out = allocate(count * 2, device);
    check(ttmi_eltwise_bf16(op, x.data, b ? y.data : nullptr, scalar, out.data, count, stream_of(device)));
    if (is_block_float(a.dtype)) out = typecast_tiles(out, DataType::BFLOAT16, a.dtype, count, device);   // the output takes input a's dtype (eltwise_binary_op.hpp:124-126)
    return like(a, std::move(out));
}

Tensor typecast(const Tensor &t, DataType dtype) {
    if (!t.on_device()) raise("TT_FATAL: Operands to copy need to be on device!");
    const int device = t.buffer.device;
    DeviceGuard guard(device);
    if (dtype == t.dtype) {
        Buffer copy_of = allocate(t.buffer.nbytes, device);
        copy(copy_of, t.buffer, t.buffer.nbytes);
        return like(t, std::move(copy_of));
    }
    auto is_float = [](DataType d) { return d == DataType::BFLOAT16 || d == DataType::FLOAT32 || is_block_float(d); };
    if (!is_float(t.dtype) || !is_float(dtype)) raise(std::string("TT_FATAL: typecast between ") + name_of(t.dtype) + " and " + name_of(dtype) + " is not supported");
    if ((is_block_float(t.dtype) || is_block_float(dtype)) && t.layout != Layout::TILE) raise("TT_FATAL: block-float tensors on device are in TILE layout");
    const uint64_t volume = t.volume();
    Buffer src = t.buffer;
    DataType from = t.dtype;
    if (is_block_float(from) && is_block_float(dtype)) {       // through bf16, which holds every block-float value exactly
        src = typecast_tiles(src, from, DataType::BFLOAT16, volume, device);
        from = DataType::BFLOAT16;
    }
    Tensor out = t;
    out.dtype = dtype;
    if (volume % 1024) {
        // dense row-major floats whose count is no multiple of 1024 (the entry point counts in tiles): the tail is padded for the call
        const uint64_t rounded = (volume + 1023) / 1024 * 1024;
        Buffer padded_src = allocate(rounded * element_bytes(from), device);
        hip_check(hipMemsetAsync(padded_src.data, 0, padded_src.nbytes, (hipStream_t)stream_of(device)), "hipMemsetAsync");
        hip_check(hipMemcpyAsync(padded_src.data, src.data, volume * element_bytes(from), hipMemcpyDeviceToDevice, (hipStream_t)stream_of(device)), "hipMemcpyAsync");
        Buffer whole = typecast_tiles(padded_src, from, dtype, rounded, device);
        out.buffer = allocate(volume * element_bytes(dtype), device);
        hip_check(hipMemcpyAsync(out.buffer.data, whole.data, out.buffer.nbytes, hipMemcpyDeviceToDevice, (hipStream_t)stream_of(device)), "hipMemcpyAsync");
        hip_check(hipStreamSynchronize((hipStream_t)stream_of(device)), "hipStreamSynchronize");      // the temporaries die here
        return out;
    }
    out.buffer = typecast_tiles(src, from, dtype, volume, device);
    return out;
}

Tensor clone(const Tensor &t, std::optional<DataType> dtype) {
    if (!t.on_device()) raise("TT_FATAL: Operands to copy need to be on device!");
    return typecast(t, dtype ? *dtype : t.dtype);
}

Tensor tilize(const Tensor &t, std::optional<DataType> dtype) {
    if (!t.on_device()) raise("TT_FATAL: Operands to tilize need to be on device!");
    if (t.layout != Layout::ROW_MAJOR) raise("TT_FATAL: Can only tilize row major data");
    const BatchHW s = batch_h_w(t.padded);
    if (s.w % 32 || (t.padded.size() > 1 && s.h % 32)) raise("TT_FATAL: tilize needs height and width to be multiples of 32");
    Tensor tiles = to_layout(t, Layout::TILE);
    if (!dtype || *dtype == tiles.dtype) return tiles;
    return typecast(tiles, *dtype);
}

// ---------------------------------------------------------------------------------------------------------------------------
// ttnn.from_torch / to_torch / to_layout / __getitem__
// ---------------------------------------------------------------------------------------------------------------------------
Tensor ttnn_from_torch_block_float(const void *data, DataType src_dtype, const Dims &shape, DataType dtype, int device) {
    // core.py:276-309 + pytensor.cpp:145-151 + tensor_impl.cpp:179-197 (pad, pack, unpack, tilize, pack) as ONE kernel
    if (shape.size() < 2) raise("ttnn.from_torch: bfloat8_b/bfloat4_b requires at least 2 dimensions!");
    if (shape.size() > 4) raise("Rank " + std::to_string(shape.size()) + " is not supported!");
    need_gpu();
    const int run_on = device >= 0 ? device : current_device();
    DeviceGuard guard(run_on);
    const BatchHW s = batch_h_w(shape);
    const size_t elem = element_bytes(src_dtype);
    Buffer host{const_cast<void *>(data), (size_t)product(shape) * elem, -1, nullptr};
    Buffer staged = moved_to(host, run_on);
    Tensor t;
    t.shape = t.padded = shape;
    t.padded[shape.size() - 2] = pad32(s.h);
    t.padded[shape.size() - 1] = pad32(s.w);
    t.dtype = dtype;
    t.layout = Layout::TILE;
    Buffer words = allocate(ttmi_tiled_size_bytes((int)dtype, s.batch, s.h, s.w), run_on);
    check(ttmi_pack_rowmajor_as_bfp_tiles((int)dtype, staged.data, (int)src_dtype, s.batch, s.h, s.w, s.w, (size_t)s.h * s.w, (uint32_t *)words.data,
                                          stream_of(run_on)));
    if (device < 0) {
        t.buffer = moved_to(words, -1);
    } else {
        hip_check(hipStreamSynchronize((hipStream_t)stream_of(run_on)), "hipStreamSynchronize");      // `staged` dies here
        t.buffer = std::move(words);
    }
    return t;
}

Tensor ttnn_to_torch(const Tensor &t) {
    if (is_block_float(t.dtype) && t.layout == Layout::TILE) {
        // one fused kernel: unpack + untilize, cropping the tile padding of the last two dimensions
        const size_t r = t.shape.size();
        Dims crop = t.padded;
        crop[r - 2] = t.shape[r - 2];
        crop[r - 1] = t.shape[r - 1];
        const BatchHW s = batch_h_w(crop);
        Tensor out;
        out.shape = t.shape; out.padded = crop; out.dtype = DataType::FLOAT32; out.layout = Layout::ROW_MAJOR;
        Tensor staged = t;
        Buffer result = through_gpu(staged, [&](const Buffer &src, int device) {
            Buffer dense = allocate((size_t)product(crop) * 4, device);
            check(ttmi_unpack_bfp_tiles_as_rowmajor((int)t.dtype, (const uint32_t *)src.data, s.batch, s.h, s.w, dense.data, TTMI_FLOAT32, stream_of(device)));
            return dense;
        });
        out.buffer = moved_to(result, -1);
        return out;
    }
    Tensor host = t.on_device() ? to_host(t) : t;
    if (host.layout != Layout::ROW_MAJOR) host = to_layout(host, Layout::ROW_MAJOR);
    return to_torch(host);
}

Tensor ttnn_to_layout(const Tensor &t, Layout layout, std::optional<DataType> dtype) {
    if (layout != Layout::ROW_MAJOR && layout != Layout::TILE) raise("Unsupported layout: " + std::to_string((int)layout));
    if (t.layout == layout && (!dtype || *dtype == t.dtype)) return t;
    if (dtype && *dtype != t.dtype) {
        // core.py:684-685, 706-711: only on the device and only towards TILE_LAYOUT (tilize with an output dtype)
        if (!t.on_device() || layout != Layout::TILE) raise(std::string("Unsupported datatype conversion to ") + name_of(*dtype));
        return typecast(t.layout != layout ? ttnn_to_layout(t, layout, std::nullopt) : t, *dtype);
    }
    if (layout == Layout::ROW_MAJOR) return to_layout(t, Layout::ROW_MAJOR);      // the tile padding stays part of the padded shape
    if (is_block_float(t.dtype)) return to_layout(t, Layout::TILE);
    const size_t rank = t.shape.size();
    if (rank < 2 || rank > 4) raise("Rank " + std::to_string(rank) + " is not supported!");
    // core.py:793: the LOGICAL tensor is padded with zeros to tile multiples and tilized (one kernel does both)
    const BatchHW s = batch_h_w(t.shape);
    const size_t elem = element_bytes(t.dtype);
    Tensor out = t;
    out.layout = Layout::TILE;
    out.padded = t.shape;
    out.padded[rank - 2] = pad32(s.h);
    out.padded[rank - 1] = pad32(s.w);
    out.buffer = through_gpu(t, [&](const Buffer &src, int device) {
        Buffer dense = src;
        if (t.padded != t.shape) {       // drop an older padding first
            const int32_t zero[4] = {0, 0, 0, 0};
            dense = window(t.dtype, src, as4(t.padded), as4(t.shape), zero, 0.f, device);
        }
        return relayout(true, dense, elem, s, device);
    });
    return out;
}

Tensor ttnn_getitem_prefix(const Tensor &t, const Dims &end) {
    require_rank4(end, "__getitem__"); require_rank4(t.shape, "__getitem__");
    if (!t.on_device()) raise("ttnn.Tensor.__getitem__: cannot slice the given tensor on the device!");
    Dims padded_end = end;
    for (int i = 0; i < 4; ++i)
        if (end[i] > t.shape[i]) raise("ttnn.Tensor.__getitem__: slice end outside the tensor");
    if (t.layout == Layout::TILE) { padded_end[2] = pad32(end[2]); padded_end[3] = pad32(end[3]); }
    Tensor out = t;
    if (padded_end != t.padded) {
        for (int i = 0; i < 4; ++i)
            if (!padded_end[i]) raise("ttnn.Tensor.__getitem__: empty slice");
        if (t.layout == Layout::TILE) {
            out = device_unpad(t, {0, 0, 0, 0}, {padded_end[0] - 1, padded_end[1] - 1, padded_end[2] - 1, padded_end[3] - 1});
        } else {
            // row-major: any width (the Tensix op wants rows that are whole 32-bit words, unpad_op.cpp:121-124; nothing here does)
            if (is_block_float(t.dtype)) raise("TT_FATAL: block-float tensors on device are in TILE layout");
            DeviceGuard guard(t.buffer.device);
            const int32_t zero[4] = {0, 0, 0, 0};
            out.buffer = window(t.dtype, t.buffer, t.padded, padded_end, zero, 0.f, t.buffer.device);
        }
    }
    out.shape = end;
    out.padded = padded_end;
    return out;
}

// ---------------------------------------------------------------------------------------------------------------------------
// Tensor files.  File = the raw bytes of `Shape` (tt_eager/tensor/types.hpp:46-63,118-121 as the x86-64 System V ABI lays it
// out), then DataType and Layout as 32-bit integers, then the element count as a 64-bit integer and the elements.
// ---------------------------------------------------------------------------------------------------------------------------
namespace {
struct FileHeader {
    uint64_t rank;                 // Shape::rank_
    uint32_t dimensions[8];        // Shape::dimensions_: the shape WITH padding, unused entries 0
    uint64_t padding_rank;         // Padding::rank_
    struct { uint64_t front, back; } pad[8];      // Padding::pad_dimensions_: back = padded - logical
    int32_t pad_value;             // Padding::pad_value_ (PadValue::Any = 0)
    int32_t struct_padding;
    int32_t dtype, layout;
    uint64_t count;                // uint32 words for block-float and UINT32, 2-byte elements for BFLOAT16 / UINT16
};
static_assert(sizeof(FileHeader) == 200, "the header is the reference's Shape object (184 bytes) plus dtype, layout and count");
size_t file_element_bytes(DataType d) { return is_block_float(d) ? 4 : element_bytes(d); }
}  // namespace

void dump_tensor(const std::string &file_name, const Tensor &t) {
    if (t.on_device()) raise("TT_THROW: Device storage isn't supported");          // serialization.cpp:113-115
    const size_t rank = t.padded.size();
    if (rank > 8) raise("TT_THROW: Shape supports up to 8 dimensions");
    FileHeader h{};
    h.rank = h.padding_rank = rank;
    for (size_t i = 0; i < rank; ++i) { h.dimensions[i] = t.padded[i]; h.pad[i].back = t.padded[i] - t.shape[i]; }
    h.dtype = (int32_t)t.dtype; h.layout = (int32_t)t.layout;
    h.count = t.buffer.nbytes / file_element_bytes(t.dtype);
    FILE *f = std::fopen(file_name.c_str(), "wb");
    if (!f) raise("Cannot open \"" + file_name + "\"");
    const bool ok = std::fwrite(&h, sizeof(h), 1, f) == 1 && (t.buffer.nbytes == 0 || std::fwrite(t.buffer.data, t.buffer.nbytes, 1, f) == 1);
    std::fclose(f);
    if (!ok) raise("Cannot write \"" + file_name + "\"");
}

Tensor load_tensor(const std::string &file_name) {
    FILE *f = std::fopen(file_name.c_str(), "rb");
    if (!f) raise("Cannot open \"" + file_name + "\"");                              // serialization.cpp:122-125
    FileHeader h{};
    if (std::fread(&h, sizeof(h), 1, f) != 1) { std::fclose(f); raise("\"" + file_name + "\" is too short to hold a tensor header"); }
    const DataType dtype = (DataType)h.dtype;
    if (h.rank > 8 || !file_element_bytes(dtype) || (h.layout != 0 && h.layout != 1)) { std::fclose(f); raise("TT_THROW: Unsupported DataType"); }
    Tensor t;
    t.dtype = dtype; t.layout = (Layout)h.layout;
    for (size_t i = 0; i < h.rank; ++i) {
        if (h.pad[i].front > h.dimensions[i] || h.pad[i].back > h.dimensions[i] - h.pad[i].front) {
            std::fclose(f);
            raise("\"" + file_name + "\": the padding of dimension " + std::to_string(i) + " exceeds the dimension");
        }
        t.padded.push_back(h.dimensions[i]);
        t.shape.push_back((uint32_t)(h.dimensions[i] - h.pad[i].front - h.pad[i].back));
    }
    // the count must be what the shape says: everything downstream indexes the buffer by the shape
    const size_t expected = storage_bytes(dtype, t.layout, t.padded);
    if (h.count > expected / file_element_bytes(dtype) || (size_t)h.count * file_element_bytes(dtype) != expected) {
        std::fclose(f);
        raise("\"" + file_name + "\": the header counts " + std::to_string(h.count) + " elements, shape " + list_of(t.padded) + " of " + name_of(dtype) + " needs " +
              std::to_string(expected / file_element_bytes(dtype)));
    }
    const size_t bytes = (size_t)h.count * file_element_bytes(dtype);
    t.buffer = allocate(bytes, -1);
    const bool ok = bytes == 0 || std::fread(t.buffer.data, bytes, 1, f) == 1;
    std::fclose(f);
    if (!ok) raise("\"" + file_name + "\" ends inside the tensor data");
    check_consistent(t, "\"" + file_name + "\"");
    return t;
}

}  // namespace ttmi::host
