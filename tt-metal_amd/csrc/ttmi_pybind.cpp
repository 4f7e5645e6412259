// pybind11 module `_ttmi`: the C ABI of include/ttmi.h with the shape of the reference's own bindings.
//
// The reference reaches this path through pybind11 modules (tt_lib._C: tt_eager/tt_lib/csrc/tt_lib_bindings_tensor_pytensor.cpp,
// tt_lib_bindings_tensor_custom_bmm_ops.cpp; ttnn._ttnn: ttnn/cpp/pybind11/operations/matmul.hpp).  This module is the
// same layer over libttmi.so: buffers are device addresses (integers, e.g. torch.Tensor.data_ptr()), `stream` is a
// hipStream_t as an integer, every failure raises RuntimeError with ttmi_last_error(), and the GIL is released around
// the calls.  Names follow the entry points they stand for.
#include <pybind11/pybind11.h>

#include <cstdint>
#include <stdexcept>
#include <string>

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

PYBIND11_MODULE(_ttmi, m) {
    m.doc() = "Block-float tensors of tt-metal / TT-NN on MI355X: pybind11 layer over the C ABI (include/ttmi.h)";

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
    m.def("eltwise",
          [](int op, uintptr_t a, uintptr_t b, float scalar, uintptr_t c, size_t count, uintptr_t stream) {
              py::gil_scoped_release release;
              check(ttmi_eltwise_bf16(op, ptr<const void>(a), ptr<const void>(b), scalar, ptr<void>(c), count, ptr<void>(stream)));
          },
          py::arg("op"), py::arg("a"), py::arg("b") = 0, py::arg("scalar") = 0.0f, py::arg("c") = 0, py::arg("count") = 0, py::arg("stream") = 0,
          "c = op(a, b | scalar), eltwise_binary_op.hpp:108-140 / eltwise_unary_op.hpp:17-90");
}
