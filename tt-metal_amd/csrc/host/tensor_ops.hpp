// Host side of the TT-NN / tt_lib surface for block-float tensors: the Tensor object and the operations on it — shape and
// padding rules, argument validation with the reference's conditions and wording, the order of conversions, dispatch to
// the C ABI of include/ttmi.h.  This is the C++ that the reference keeps in tt_eager/tensor/ (tensor.cpp, tensor_impl.cpp),
// tt_eager/tt_lib/csrc/tt_lib_bindings_tensor_pytensor.cpp and tt_eager/tt_dnn/op_library/bmm/bmm_op.cpp; the Python layers
// above it (ttnn/, tt_lib/) only adapt signatures, as ttnn/ttnn/decorators.py does over ttnn._ttnn.
//
// Memory and the stream come from whoever embeds this layer (Runtime): in this repository torch's allocator and torch's
// current stream.  Nothing here computes on the CPU; without a GPU every conversion raises.
#pragma once
#include <cstddef>
#include <cstdint>
#include <functional>
#include <memory>
#include <optional>
#include <string>
#include <vector>

namespace ttmi::host {

enum class DataType : int { BFLOAT16 = 0, FLOAT32 = 1, UINT32 = 2, BFLOAT8_B = 3, BFLOAT4_B = 4, UINT16 = 6, INVALID = 7 };   // tt_eager/tensor/types.hpp:26-34
enum class Layout : int { ROW_MAJOR = 0, TILE = 1, INVALID = 2 };                                                          // types.hpp:24
using Dims = std::vector<uint32_t>;

// A block of memory and whoever keeps it alive.  device < 0: host memory.
struct Buffer {
    void *data = nullptr;
    size_t nbytes = 0;
    int device = -1;
    std::shared_ptr<void> owner;
};

// What the embedding provides.
struct Runtime {
    std::function<Buffer(size_t nbytes, int device)> allocate;     // uninitialised memory, 256-byte aligned on the device
    std::function<void *(int device)> stream;                      // the stream to launch on (hipStream_t)
    std::function<bool()> gpu_available;
};
void set_runtime(Runtime runtime);

struct Tensor {
    Buffer buffer;
    Dims shape;        // logical shape
    Dims padded;       // legacy shape: with tile padding
    DataType dtype = DataType::INVALID;
    Layout layout = Layout::INVALID;
    bool allocated() const { return buffer.data != nullptr || volume() == 0; }
    bool on_device() const { return buffer.device >= 0; }
    uint64_t volume() const;                                       // of the padded shape
};

bool is_block_float(DataType dtype);
size_t element_bytes(DataType dtype);                              // of the dense formats
size_t storage_bytes(DataType dtype, Layout layout, const Dims &padded);
const char *name_of(DataType dtype);
const char *name_of(Layout layout);

// ---- tt_lib.tensor.Tensor ------------------------------------------------------------------------------------------------
// Tensor(torch_tensor, data_type): `data` is host memory holding the elements in `dtype`'s storage type (fp32 for block-float:
// tt_lib_bindings_tensor_pytensor.cpp:78-85), row-major; the result is a host tensor declared ROW_MAJOR (:145-151).
Tensor from_host(const void *data, const Dims &shape, DataType dtype);
Tensor wrap(Buffer buffer, const Dims &shape, const Dims &padded, DataType dtype, Layout layout);
Tensor to_layout(const Tensor &t, Layout target);                  // Tensor::to(Layout), tensor_impl.hpp:158-171, tensor_impl.cpp:179-197
Tensor to_device(const Tensor &t, int device);
Tensor to_host(const Tensor &t);
Tensor reshape(const Tensor &t, const Dims &logical, const Dims &padded);
Tensor to_torch(const Tensor &t);                                  // pytensor.cpp:354-412: host buffer of the padded shape, fp32 for block-float
Tensor pad(const Tensor &t, const Dims &output_shape, const Dims &input_start, float pad_value);      // tensor.cpp:204-224
Tensor unpad(const Tensor &t, const Dims &start, const Dims &end);                                     // tensor.cpp:226-230
Tensor pad_to_tile(const Tensor &t, float pad_value);                                                  // tensor.cpp:232-246
Tensor unpad_from_tile(const Tensor &t, const Dims &output_shape);                                     // tensor.cpp:248-260
Tensor device_unpad(const Tensor &t, const Dims &start, const Dims &end);                              // unpad_op.cpp:95-125

// ---- matmul family (bmm_op.cpp:518-539, 828-1049) ---------------------------------------------------------------------------
// untilize_out: the output is a ROW_MAJOR bf16 tensor of the padded shape instead of a TILE one (bmm_op.cpp:1069; :536-538, :865-867)
Tensor matmul(const Tensor &a, const Tensor &b, bool bcast_batch, const Tensor *bias, int activation, std::optional<DataType> output_dtype,
              const std::string &op, bool untilize_out = false);
// act(a . b_gate) * (a . b_up) in one launch (ttmi_matmul_bfp_gated): what a gated MLP issues as linear(activation), linear, mul
Tensor matmul_gated(const Tensor &a, const Tensor &b_gate, const Tensor &b_up, int activation, std::optional<DataType> output_dtype,
                    const std::string &op);
// ttnn.matmul / ttnn.linear (ttnn/cpp/ttnn/operations/matmul.hpp:39-62, ttnn/ttnn/operations/matmul.py:200-220)
Tensor ttnn_matmul(const std::string &operation_name, const Tensor &a, const Tensor &b, const Tensor *bias,
                   const std::optional<std::string> &activation, std::optional<DataType> dtype);
int activation_code(const std::optional<std::string> &activation);

// ---- elementwise, dtype changes ---------------------------------------------------------------------------------------------
Tensor eltwise(int op, const Tensor &a, const Tensor *b, float scalar, const std::string &name);      // eltwise_binary_op.hpp:108-140
Tensor typecast(const Tensor &t, DataType dtype);                                                      // copy_op.hpp:44
Tensor clone(const Tensor &t, std::optional<DataType> dtype);                                          // copy_op.hpp:42
Tensor tilize(const Tensor &t, std::optional<DataType> dtype);                                         // tilize_op.hpp:71-73

// ---- ttnn.from_torch / to_torch / to_layout / __getitem__ (ttnn/ttnn/operations/core.py) ------------------------------------
// from_torch for block-float: data is host fp32 or bf16 (src_dtype), logical shape `shape`; one fused pad + tilize + pack.
Tensor ttnn_from_torch_block_float(const void *data, DataType src_dtype, const Dims &shape, DataType dtype, int device);
Tensor ttnn_to_torch(const Tensor &t);                             // host buffer of the LOGICAL shape (the last two dims cropped), fp32 for block-float
Tensor ttnn_to_layout(const Tensor &t, Layout layout, std::optional<DataType> dtype);
Tensor ttnn_getitem_prefix(const Tensor &t, const Dims &end);      // rank 4: keeps [0, end) in every dimension

// ---- tensor files (tt_eager/tensor/serialization.cpp:86-141) ----------------------------------------------------------------
void dump_tensor(const std::string &file_name, const Tensor &t);
Tensor load_tensor(const std::string &file_name);

}  // namespace ttmi::host
