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
#include <migraphx/program.hpp>

namespace migraphx {

// src/include/migraphx/onnx.hpp:62-76
program parse_onnx(const std::string& filename);
program parse_onnx_buffer(const std::string& buffer);
program parse_onnx_buffer(const void* data, std::size_t size);

} // namespace migraphx
#endif
