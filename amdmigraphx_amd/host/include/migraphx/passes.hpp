// Passes on the quantized-GEMM path, and the user-facing quantization entry points.
#ifndef MIGRAPHX_GUARD_PASSES_HPP
#define MIGRAPHX_GUARD_PASSES_HPP

#include <functional>
#include <memory>
#include <string>
#include <unordered_set>
#include <vector>
#include <migraphx/pass.hpp>
#include <migraphx/program.hpp>

namespace migraphx {

// Remove instructions whose result no module output depends on (src/dead_code_elimination.cpp).
struct dead_code_elimination
{
    std::string name() const { return "dead_code_elimination"; }
    void apply(module& m) const;
};

// Turn dequantizelinear -> dot into quant_dot -> dequantizelinear, dequantizelinear -> convolution
// into quant_convolution -> dequantizelinear, and drop the fake-quantization pairs that remain
// (src/simplify_qdq.cpp:126-289, :498-594, :642-670); with use_mx_quant also the block-scale
// branch (:290-357).  The concat / reused-quantizelinear rewrites are not part of this build.
struct simplify_qdq
{
    bool remove_qdq_only = false;
    // also rewrite dot(DQ(a, block scales), DQ(b, block scales)) to the four-input quant_dot
    // (simplify_qdq.hpp:42, set by a target whose hardware has block-scaled matrix instructions)
    bool use_mx_quant = false;
    std::string name() const { return "simplify_qdq"; }
    void apply(module& m) const;
};

// Wrap every quantizable input of the named instructions in a `capture` operator
// (src/quantize_8bits.cpp:98-126).
struct capture_arguments_pass
{
    std::unordered_set<std::string> ins_names = {"dot", "convolution"};
    std::function<void(std::size_t, std::vector<argument>)> f{};
    std::size_t* param_index = nullptr;
    std::string name() const { return "capture_arguments"; }
    void apply(module& m) const;
};

// Replace each `capture` by quantizelinear -> dequantizelinear with the calibrated scale
// (src/quantize_8bits.cpp:52-96).
struct quantize_8bits_pass
{
    shape::type_t precision = shape::int8_type;
    std::vector<std::pair<float, float>> quant_params;
    std::string name() const { return "quantize_8bits"; }
    void apply(module& m) const;
};

// Fake-quantize constant float inputs of dot to 4 bits, per tensor
// (src/quantize_int4.cpp:38-103).
struct quantize_int4_pass
{
    std::string name() const { return "quantize_int4"; }
    void apply(module& m) const;
};

// src/quantization.cpp:88-210
void quantize_int8(program& prog,
                   const target& t,
                   const std::vector<parameter_map>& calibration,
                   const std::unordered_set<std::string>& ins_names = {"dot", "convolution"});
void quantize_fp8(program& prog, const target& t, const std::vector<parameter_map>& calibration);
void quantize_int4_weights(program& prog);

namespace op {
namespace builder {
// The instructions the ONNX MatMulNBits node expands to (src/onnx/parse_matmulnbits.cpp:42-159):
// b is uint8 [N, ceil(K/block), block/2], scales has N*ceil(K/block) elements, zp (optional, may be
// m.end()) is uint8 [N * ceil(ceil(K/block)/2)] of packed 4-bit zero points.  Returns dot(a, B^T).
instruction_ref matmulnbits(module& m,
                            instruction_ref a,
                            instruction_ref b,
                            instruction_ref scales,
                            instruction_ref zp,
                            std::size_t n,
                            std::size_t k,
                            std::size_t block_size);
} // namespace builder
} // namespace op

} // namespace migraphx
#endif
