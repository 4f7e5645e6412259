// pybind11 module `_ttmi`: the C ABI of include/ttmi.h with the shape of the reference's own bindings.
//
// Two layers.  (1) Tensor and the operations on it (host/tensor_ops.hpp): shapes, validation, conversion sequences and
// dispatch in C++, as the reference keeps them in tt_lib._C / ttnn._ttnn; the Python packages ttnn/ and tt_lib/ are
// signature shims over this.  Memory and the stream come from Python callbacks (torch's allocator, torch's current
// stream).  (2) The entry points of the C ABI on raw device addresses, for callers that manage their own buffers.
//
// The reference reaches this path through pybind11 modules (tt_lib._C: tt_eager/tt_lib/csrc/tt_lib_bindings_tensor_pytensor.cpp,
// tt_lib_bindings_tensor_custom_bmm_ops.cpp; ttnn._ttnn: ttnn/cpp/pybind11/operations/matmul.hpp).  This module is the
// same layer over libttmi.so: buffers are device addresses (integers, e.g. torch.Tensor.data_ptr()), `stream` is a
// hipStream_t as an integer, every failure raises RuntimeError with ttmi_last_error(), and the GIL is released around
// the calls.  Names follow the entry points they stand for.
#include <pybind11/functional.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstdint>
#include <stdexcept>
#include <string>

#include "host/tensor_ops.hpp"
#include "ttmi.h"

namespace py = pybind11;

namespace {

template <typename T> T *ptr(uintptr_t address) { return reinterpret_cast<T *>(address); }

void check(int status) {
    if (status != TTMI_OK) throw std::runtime_error(std::string(ttmi_last_error()));
}

int activation_code(const py::object &activation) {   // ttnn/ttnn/operations/matmul.py:59-63
    if (activation.is_none()) return TTMI_ACT_NONE;
    const std::string name = py::cast<std::string>(activation);
    if (name == "relu") return TTMI_ACT_RELU;
    if (name == "gelu") return TTMI_ACT_GELU;
    if (name == "silu") return TTMI_ACT_SILU;
    throw std::runtime_error(name + " is not supported as activation function. Use one of these instead: ['relu', 'gelu', 'silu']");
}

}  // namespace

namespace host = ttmi::host;

// a Python object (a torch tensor) as the owner of a Buffer; dropped under the GIL
std::shared_ptr<void> keep_alive(py::object object) {
    return std::shared_ptr<void>(new py::object(std::move(object)), [](void *p) {
        py::gil_scoped_acquire gil;
        delete static_cast<py::object *>(p);
    });
}
py::object owner_of(const host::Tensor &t) {
    if (!t.buffer.owner) return py::none();
    return *static_cast<py::object *>(t.buffer.owner.get());
}
std::optional<host::DataType> optional_dtype(const py::object &dtype) {
    if (dtype.is_none()) return std::nullopt;
    return (host::DataType)py::cast<int>(dtype);
}
// Runs a host-layer operation (launches, synchronising copies) with the GIL released; the Runtime callbacks re-acquire it.
// Arguments are converted from Python before, the result is converted after.
template <typename F> auto unlocked(F &&f) {
    py::gil_scoped_release release;
    return f();
}
const host::Tensor *optional_tensor(const py::object &t) { return t.is_none() ? nullptr : &py::cast<const host::Tensor &>(t); }

void bind_tensor_layer(py::module_ &m) {
    py::class_<host::Tensor>(m, "Tensor", py::module_local(), "Shape with and without tile padding, data type, layout and a buffer on the host or on a GPU")
        .def_property_readonly("shape", [](const host::Tensor &t) { return py::tuple(py::cast(t.shape)); })
        .def_property_readonly("padded_shape", [](const host::Tensor &t) { return py::tuple(py::cast(t.padded)); })
        .def_property_readonly("dtype", [](const host::Tensor &t) { return (int)t.dtype; })
        .def_property_readonly("layout", [](const host::Tensor &t) { return (int)t.layout; })
        .def_property_readonly("device", [](const host::Tensor &t) { return t.buffer.device; })
        .def_property_readonly("nbytes", [](const host::Tensor &t) { return t.buffer.nbytes; })
        .def_property_readonly("data_ptr", [](const host::Tensor &t) { return (uintptr_t)t.buffer.data; })
        .def_property_readonly("storage", &owner_of, "the object that owns the memory (a flat torch.uint8 tensor)")
        .def("volume", &host::Tensor::volume);

    m.def("set_runtime",
          [](py::function allocate, py::function stream, py::function gpu_available) {
              host::Runtime rt;
              // the operations below run with the GIL released; the callbacks are Python and take it back for their own duration
              rt.allocate = [allocate](size_t nbytes, int device) {
                  py::gil_scoped_acquire gil;
                  py::object storage = allocate(nbytes, device);                  // flat uint8 tensor on that device (-1: host)
                  host::Buffer b;
                  b.data = reinterpret_cast<void *>(py::cast<uintptr_t>(storage.attr("data_ptr")()));
                  b.nbytes = nbytes;
                  b.device = device;
                  b.owner = keep_alive(std::move(storage));
                  return b;
              };
              rt.stream = [stream](int device) { py::gil_scoped_acquire gil; return reinterpret_cast<void *>(py::cast<uintptr_t>(stream(device))); };
              rt.gpu_available = [gpu_available]() { py::gil_scoped_acquire gil; return py::cast<bool>(gpu_available()); };
              host::set_runtime(std::move(rt));
              // the callbacks are Python objects: they go before the interpreter does
              static bool registered = false;
              if (!registered) {
                  py::module_::import("atexit").attr("register")(py::cpp_function([]() { host::set_runtime(host::Runtime{}); }));
                  registered = true;
              }
          },
          py::arg("allocate"), py::arg("stream"), py::arg("gpu_available"),
          "allocate(nbytes, device) -> flat uint8 tensor (device -1: host); stream(device) -> hipStream_t as an integer; gpu_available() -> bool");

    m.def("wrap",
          [](py::object storage, uintptr_t data, size_t nbytes, int device, host::Dims shape, host::Dims padded, int dtype, int layout) {
              host::Buffer b;
              b.data = reinterpret_cast<void *>(data); b.nbytes = nbytes; b.device = device; b.owner = keep_alive(std::move(storage));
              return host::wrap(std::move(b), shape, padded, (host::DataType)dtype, (host::Layout)layout);
          },
          "a Tensor over memory that a Python object owns");
    m.def("from_host", [](uintptr_t data, host::Dims shape, int dtype) { return unlocked([&] { return host::from_host(reinterpret_cast<const void *>(data), shape, (host::DataType)dtype); }); },
          "tt_lib.tensor.Tensor(torch_tensor, data_type), tt_lib_bindings_tensor_pytensor.cpp:26-167");
    const auto no_gil = py::call_guard<py::gil_scoped_release>();
    m.def("to_layout", [](const host::Tensor &t, int layout) { return host::to_layout(t, (host::Layout)layout); }, no_gil);
    m.def("to_device", &host::to_device, no_gil);
    m.def("to_host", &host::to_host, no_gil);
    m.def("reshape", &host::reshape);
    m.def("to_torch", &host::to_torch, no_gil);
    m.def("pad", &host::pad, no_gil);
    m.def("unpad", &host::unpad, no_gil);
    m.def("pad_to_tile", &host::pad_to_tile, no_gil);
    m.def("unpad_from_tile", &host::unpad_from_tile, no_gil);
    m.def("device_unpad", &host::device_unpad, no_gil);
    m.def("matmul",
          [](const host::Tensor &a, const host::Tensor &b, bool bcast_batch, const py::object &bias, int activation, const py::object &output_dtype,
             const std::string &op, bool untilize_out) {
              const host::Tensor *bias_tensor = optional_tensor(bias);
              const std::optional<host::DataType> dtype = optional_dtype(output_dtype);
              return unlocked([&] { return host::matmul(a, b, bcast_batch, bias_tensor, activation, dtype, op, untilize_out); });
          },
          py::arg("a"), py::arg("b"), py::arg("bcast_batch"), py::arg("bias") = py::none(), py::arg("activation") = 0, py::arg("output_dtype") = py::none(),
          py::arg("op") = "matmul", py::arg("untilize_out") = false, "tt::operations::primary::matmul, tt_eager/tt_dnn/op_library/bmm/bmm_op.cpp:828-1049");
    m.def("matmul_gated",
          [](const host::Tensor &a, const host::Tensor &b_gate, const host::Tensor &b_up, int activation, const py::object &output_dtype, const std::string &op) {
              const std::optional<host::DataType> dtype = optional_dtype(output_dtype);
              return unlocked([&] { return host::matmul_gated(a, b_gate, b_up, activation, dtype, op); });
          },
          py::arg("a"), py::arg("b_gate"), py::arg("b_up"), py::arg("activation") = 0, py::arg("output_dtype") = py::none(), py::arg("op") = "gated_linear",
          "act(a . b_gate) * (a . b_up) in one launch: linear(activation) + linear + mul of a gated MLP (models/demos/mistral7b/tt/mistral_mlp.py:43-82)");
    m.def("ttnn_matmul",
          [](const std::string &name, const host::Tensor &a, const host::Tensor &b, const py::object &bias, const py::object &activation,
             const py::object &dtype) {
              std::optional<std::string> act;
              if (!activation.is_none()) act = py::cast<std::string>(py::str(activation));
              const host::Tensor *bias_tensor = optional_tensor(bias);
              const std::optional<host::DataType> out_dtype = optional_dtype(dtype);
              return unlocked([&] { return host::ttnn_matmul(name, a, b, bias_tensor, act, out_dtype); });
          },
          py::arg("operation_name"), py::arg("a"), py::arg("b"), py::arg("bias") = py::none(), py::arg("activation") = py::none(), py::arg("dtype") = py::none(),
          "ttnn.matmul / ttnn.linear, ttnn/cpp/ttnn/operations/matmul.hpp:44-214");
    m.def("activation_code", [](const py::object &activation) {
        std::optional<std::string> act;
        if (!activation.is_none()) act = py::cast<std::string>(py::str(activation));
        return host::activation_code(act);
    });
    m.def("eltwise",
          [](int op, const host::Tensor &a, const py::object &b, float scalar, const std::string &name) {
              const host::Tensor *other = optional_tensor(b);
              return unlocked([&] { return host::eltwise(op, a, other, scalar, name); });
          },
          py::arg("op"), py::arg("a"), py::arg("b") = py::none(), py::arg("scalar") = 0.0f, py::arg("name") = "eltwise");
    m.def("typecast", [](const host::Tensor &t, int dtype) { return host::typecast(t, (host::DataType)dtype); }, no_gil);
    m.def("clone", [](const host::Tensor &t, const py::object &dtype) { const auto d = optional_dtype(dtype); return unlocked([&] { return host::clone(t, d); }); });
    m.def("tilize", [](const host::Tensor &t, const py::object &dtype) { const auto d = optional_dtype(dtype); return unlocked([&] { return host::tilize(t, d); }); });
    m.def("ttnn_from_torch_block_float",
          [](uintptr_t data, int src_dtype, host::Dims shape, int dtype, int device) {
              return unlocked([&] { return host::ttnn_from_torch_block_float(reinterpret_cast<const void *>(data), (host::DataType)src_dtype, shape, (host::DataType)dtype, device); });
          },
          "ttnn.from_torch(dtype=bfloat8_b|bfloat4_b, layout=TILE_LAYOUT), ttnn/ttnn/operations/core.py:245-311, as one fused kernel");
    m.def("ttnn_to_torch", &host::ttnn_to_torch, no_gil);
    m.def("ttnn_to_layout", [](const host::Tensor &t, int layout, const py::object &dtype) {
        const auto d = optional_dtype(dtype);
        return unlocked([&] { return host::ttnn_to_layout(t, (host::Layout)layout, d); });
    });
    m.def("ttnn_getitem_prefix", &host::ttnn_getitem_prefix, no_gil);
    m.def("dump_tensor", &host::dump_tensor, no_gil);
    m.def("load_tensor", &host::load_tensor, no_gil);
}

#ifndef TTMI_PYBIND_NAME
#define TTMI_PYBIND_NAME _ttmi      // the test build (against libttmi_test.so) is _ttmi_test
#endif
PYBIND11_MODULE(TTMI_PYBIND_NAME, m) {
    m.doc() = "Block-float tensors of tt-metal / TT-NN on MI355X: the host layer (Tensor and its operations) and the C ABI (include/ttmi.h)";
    bind_tensor_layer(m);

    m.attr("BFLOAT16") = (int)TTMI_BFLOAT16;
    m.attr("FLOAT32") = (int)TTMI_FLOAT32;
    m.attr("BFLOAT8_B") = (int)TTMI_BFLOAT8_B;
    m.attr("BFLOAT4_B") = (int)TTMI_BFLOAT4_B;
    m.attr("ROW_MAJOR") = (int)TTMI_ROW_MAJOR;
    m.attr("TILE") = (int)TTMI_TILE;

    m.def("version", []() { return std::string(ttmi_version()); });
    m.def("tile_size", &ttmi_tile_size, py::arg("dtype"), "tile_size(DataFormat), tt_metal/common/tt_backend_api_types.hpp:109-132");
    m.def("tiled_size_bytes", &ttmi_tiled_size_bytes, py::arg("dtype"), py::arg("batch"), py::arg("h"), py::arg("w"),
          "compute_buffer_size for TILE layout, tt_eager/tensor/tensor_utils.hpp:33-49");

    m.def("pack_fp32_vec_as_bfp_tiles",
          [](int fmt, uintptr_t src, size_t n_tiles, bool row_major_input, uintptr_t dst, uintptr_t stream) {
              py::gil_scoped_release release;
              check(ttmi_pack_fp32_vec_as_bfp_tiles(fmt, ptr<const float>(src), n_tiles, row_major_input, ptr<uint32_t>(dst), ptr<void>(stream)));
          },
          py::arg("fmt"), py::arg("src"), py::arg("n_tiles"), py::arg("row_major_input"), py::arg("dst"), py::arg("stream") = 0,
          "pack_fp32_vec_as_bfp8_tiles / pack_fp32_vec_as_bfp4_tiles, tt_metal/common/bfloat8.hpp:102, bfloat4.hpp:23");
    m.def("unpack_bfp_tiles_into_float_vec",
          [](int fmt, uintptr_t words, size_t n_tiles, bool row_major_output, uintptr_t dst, uintptr_t stream) {
              py::gil_scoped_release release;
              check(ttmi_unpack_bfp_tiles_into_float_vec(fmt, ptr<const uint32_t>(words), n_tiles, row_major_output, ptr<float>(dst), ptr<void>(stream)));
          },
          py::arg("fmt"), py::arg("words"), py::arg("n_tiles"), py::arg("row_major_output"), py::arg("dst"), py::arg("stream") = 0,
          "unpack_bfp8_tiles_into_float_vec / unpack_bfp4_tiles_into_float_vec, bfloat8.hpp:175, bfloat4.hpp:33");

    m.def("from_torch",
          [](int dtype, uintptr_t src, int src_dtype, uint32_t batch, uint32_t h, uint32_t w, uint64_t row_stride, uint64_t batch_stride,
             uintptr_t dst, uintptr_t stream) {
              py::gil_scoped_release release;
              check(ttmi_pack_rowmajor_as_bfp_tiles(dtype, ptr<const void>(src), src_dtype, batch, h, w, row_stride, batch_stride,
                                                    ptr<uint32_t>(dst), ptr<void>(stream)));
          },
          py::arg("dtype"), py::arg("src"), py::arg("src_dtype"), py::arg("batch"), py::arg("h"), py::arg("w"), py::arg("row_stride"),
          py::arg("batch_stride"), py::arg("dst"), py::arg("stream") = 0,
          "ttnn.from_torch(dtype=bfloat8_b|bfloat4_b, layout=TILE_LAYOUT) on device memory, ttnn/ttnn/operations/core.py:245-311");
    m.def("to_torch",
          [](int dtype, uintptr_t words, uint32_t batch, uint32_t h, uint32_t w, uintptr_t dst, int dst_dtype, uintptr_t stream) {
              py::gil_scoped_release release;
              check(ttmi_unpack_bfp_tiles_as_rowmajor(dtype, ptr<const uint32_t>(words), batch, h, w, ptr<void>(dst), dst_dtype, ptr<void>(stream)));
          },
          py::arg("dtype"), py::arg("words"), py::arg("batch"), py::arg("h"), py::arg("w"), py::arg("dst"), py::arg("dst_dtype") = (int)TTMI_FLOAT32,
          py::arg("stream") = 0, "ttnn.to_torch of a block-float tensor, ttnn/ttnn/operations/core.py:336-394");

    m.def("tilize",
          [](uintptr_t src, uint32_t elem_size, uint32_t batch, uint32_t h, uint32_t w, uintptr_t dst, uintptr_t stream) {
              py::gil_scoped_release release;
              check(ttmi_tilize(ptr<const void>(src), elem_size, batch, h, w, ptr<void>(dst), ptr<void>(stream)));
          },
          py::arg("src"), py::arg("elem_size"), py::arg("batch"), py::arg("h"), py::arg("w"), py::arg("dst"), py::arg("stream") = 0,
          "convert_layout to 4-face tiles, tt_metal/common/test_tiles.hpp:177-213");
    m.def("untilize",
          [](uintptr_t src, uint32_t elem_size, uint32_t batch, uint32_t h, uint32_t w, uintptr_t dst, uintptr_t stream) {
              py::gil_scoped_release release;
              check(ttmi_untilize(ptr<const void>(src), elem_size, batch, h, w, ptr<void>(dst), ptr<void>(stream)));
          },
          py::arg("src"), py::arg("elem_size"), py::arg("batch"), py::arg("h"), py::arg("w"), py::arg("dst"), py::arg("stream") = 0,
          "convert_layout back to row-major, tt_metal/common/test_tiles.hpp:92-118");

    m.def("matmul_workspace_bytes", &ttmi_matmul_bfp_workspace_bytes, py::arg("batch"), py::arg("m"), py::arg("k"), py::arg("n"), py::arg("b_fmt"));
    // ttnn::operations::matmul::linear (ttnn/cpp/ttnn/operations/matmul.hpp:117-214): matmul is linear without bias and activation
    m.def("linear",
          [](uintptr_t a, int a_layout, uintptr_t b, int b_dtype, uint32_t batch, uint32_t b_batch, uint32_t mm, uint32_t k, uint32_t n,
             uintptr_t bias, const py::object &activation, uintptr_t c, int c_layout, int c_dtype, uintptr_t workspace, size_t workspace_bytes,
             uintptr_t stream) {
              const int act = activation_code(activation);
              if (act != TTMI_ACT_NONE && b_batch != 1) throw std::runtime_error("Cannot use activation with batched input b");   // matmul.py:215-216
              py::gil_scoped_release release;
              check(ttmi_matmul_bfp(ptr<const void>(a), a_layout, ptr<const uint32_t>(b), b_dtype, batch, b_batch, mm, k, n, ptr<const void>(bias), act,
                                    ptr<void>(c), c_layout, c_dtype, ptr<void>(workspace), workspace_bytes, ptr<void>(stream)));
          },
          py::arg("a"), py::arg("a_layout"), py::arg("b"), py::arg("b_dtype"), py::arg("batch"), py::arg("b_batch"), py::arg("m"), py::arg("k"),
          py::arg("n"), py::arg("bias") = 0, py::arg("activation") = py::none(), py::arg("c") = 0, py::arg("c_layout") = (int)TTMI_TILE,
          py::arg("c_dtype") = (int)TTMI_BFLOAT16, py::arg("workspace") = 0, py::arg("workspace_bytes") = 0, py::arg("stream") = 0,
          "ttnn.linear / ttnn.matmul with block-float weights, ttnn/cpp/ttnn/operations/matmul.hpp:44-214");
    // ttnn.mul / add / sub and gelu / relu / silu on bf16 tensors of equal shape (ttnn/ttnn/operations/binary.py:321-424)
    m.def("eltwise_bf16",
          [](int op, uintptr_t a, uintptr_t b, float scalar, uintptr_t c, size_t count, uintptr_t stream) {
              py::gil_scoped_release release;
              check(ttmi_eltwise_bf16(op, ptr<const void>(a), ptr<const void>(b), scalar, ptr<void>(c), count, ptr<void>(stream)));
          },
          py::arg("op"), py::arg("a"), py::arg("b") = 0, py::arg("scalar") = 0.0f, py::arg("c") = 0, py::arg("count") = 0, py::arg("stream") = 0,
          "c = op(a, b | scalar), eltwise_binary_op.hpp:108-140 / eltwise_unary_op.hpp:17-90");
}
