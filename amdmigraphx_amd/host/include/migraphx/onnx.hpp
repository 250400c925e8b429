// ONNX front end for the quantized-GEMM path: reads a ModelProto from its protobuf wire format and
// builds a program from the nodes that path consists of -- MatMul, MatMulNBits (com.microsoft),
// QLinearMatMul, Conv, QuantizeLinear, DequantizeLinear (per tensor, per axis, blocked), the float binary operators,
// Transpose, Reshape, Identity.  Follows src/onnx/onnx_parser.cpp (graph inputs that are not
// initializers become parameters in input order, initializers become literals, graph outputs the
// return) and the node parsers named at each operator in onnx.cpp.  Any other operator type
// throws.
#ifndef MIGRAPHX_GUARD_ONNX_HPP
#define MIGRAPHX_GUARD_ONNX_HPP

#include <string>
#include <unordered_map>
#include <vector>
#include <migraphx/program.hpp>

namespace migraphx {

// src/include/migraphx/onnx.hpp:34-60, the static-shape part
struct onnx_options
{
    // a dimension the file leaves open takes this size (0: the reference's default of 1)
    std::size_t default_dim_value = 0;
    // dimensions given here replace the ones the file declares for that input
    std::unordered_map<std::string, std::vector<std::size_t>> map_input_dims;
};

// src/include/migraphx/onnx.hpp:62-76
program parse_onnx(const std::string& filename, const onnx_options& options = onnx_options{});
program parse_onnx_buffer(const std::string& buffer, const onnx_options& options = onnx_options{});
program parse_onnx_buffer(const void* data, std::size_t size, const onnx_options& options = onnx_options{});

} // namespace migraphx
#endif
