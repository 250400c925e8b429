// Test-only CPU target "oracle": evaluates the operators of the quantized-GEMM path with the C
// oracle (oracle/ref_oracle.c), standing in for the reference's `ref` target in the parity tests.
// It lives under tests/ and is linked into the test programs only; no library of the product
// knows it.
#ifndef TESTS_CPP_ORACLE_TARGET_HPP
#define TESTS_CPP_ORACLE_TARGET_HPP

#include <string>
#include <vector>
#include <migraphx/context.hpp>
#include <migraphx/operation.hpp>
#include <migraphx/pass.hpp>
#include <migraphx/target.hpp>

namespace oracle {

struct context
{
    void finish() const {}
};

// the operator that evaluates `op` with the oracle
migraphx::operation wrap(const migraphx::operation& op);

struct lowering
{
    std::string name() const { return "oracle::lowering"; }
    void apply(migraphx::module& m) const;
};

struct target
{
    std::string name() const { return "oracle"; }
    std::vector<migraphx::pass> get_passes(migraphx::context&, const migraphx::compile_options&) const;
    migraphx::context get_context() const { return context{}; }
};

} // namespace oracle
#endif
