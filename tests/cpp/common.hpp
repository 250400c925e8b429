// Helpers shared by the host-layer test programs.
#ifndef TESTS_CPP_COMMON_HPP
#define TESTS_CPP_COMMON_HPP

#include <cmath>
#include <cstdint>
#include <map>
#include <random>
#include <sstream>
#include <string>
#include <vector>
#include <migraphx/ops.hpp>
#include <migraphx/passes.hpp>
#include <migraphx/program.hpp>
#include <migraphx/register_target.hpp>

namespace testutil {

using migraphx::argument;
using migraphx::instruction_ref;
using migraphx::literal;
using migraphx::make_op;
using migraphx::module;
using migraphx::program;
using migraphx::shape;

// compile a copy of p for the named target and run it on host inputs; results come back on the host
inline std::vector<argument> run_on(const std::string& target_name,
                                    const program& p,
                                    const migraphx::parameter_map& host_params,
                                    bool offload_copy = false)
{
    auto t       = migraphx::make_target(target_name);
    program copy = p;
    migraphx::compile_options opts;
    opts.offload_copy = offload_copy;
    copy.compile(t, opts);
    migraphx::parameter_map params;
    for(const auto& kv : host_params)
        params[kv.first] = offload_copy ? kv.second : t.copy_to(kv.second);
    auto res = copy.eval(params);
    copy.finish();
    std::vector<argument> out;
    for(auto& r : res)
        out.push_back(offload_copy ? r : t.copy_from(r));
    return out;
}

// expression tree of a module's results: independent of instruction order and dead code
inline std::string expr(instruction_ref ins, std::map<const migraphx::instruction*, std::string>& memo)
{
    auto it = memo.find(&*ins);
    if(it != memo.end())
        return it->second;
    std::stringstream ss;
    if(ins->name() == "@literal")
        ss << "lit{" << ins->get_literal() << ":" << ins->get_shape() << "}";
    else if(ins->name() == "@param")
        ss << migraphx::any_cast<migraphx::builtin::param>(ins->get_operator()).parameter;
    else
    {
        ss << ins->get_operator() << "(";
        for(std::size_t i = 0; i < ins->inputs().size(); i++)
            ss << (i == 0 ? "" : ",") << expr(ins->inputs()[i], memo);
        ss << ")->" << ins->get_shape();
    }
    memo[&*ins] = ss.str();
    return ss.str();
}

inline std::string canonical(const module& m)
{
    std::map<const migraphx::instruction*, std::string> memo;
    std::string r;
    for(auto i : m.get_returns())
        r += expr(i, memo) + ";";
    return r;
}

inline std::size_t count_ops(const module& m, const std::string& name)
{
    std::size_t n = 0;
    for(auto it = m.begin(); it != m.end(); ++it)
        n += it->name() == name ? 1 : 0;
    return n;
}

template <class T>
std::vector<T> uniform_ints(std::size_t n, int lo, int hi, unsigned seed)
{
    std::mt19937 g(seed);
    std::uniform_int_distribution<int> d(lo, hi);
    std::vector<T> v(n);
    for(auto& x : v)
        x = static_cast<T>(d(g));
    return v;
}

inline std::vector<float> normal_floats(std::size_t n, float sigma, unsigned seed)
{
    std::mt19937 g(seed);
    std::normal_distribution<float> d(0.0f, sigma);
    std::vector<float> v(n);
    for(auto& x : v)
        x = d(g);
    return v;
}

inline std::vector<float> uniform_floats(std::size_t n, float lo, float hi, unsigned seed)
{
    std::mt19937 g(seed);
    std::uniform_real_distribution<float> d(lo, hi);
    std::vector<float> v(n);
    for(auto& x : v)
        x = d(g);
    return v;
}

// raw bytes equal
inline bool same_bytes(const argument& x, const argument& y)
{
    return x.get_shape().lens() == y.get_shape().lens() and
           x.get_shape().type() == y.get_shape().type() and
           std::memcmp(x.data(), y.data(), x.get_shape().bytes()) == 0;
}

// largest |x - y| / max(|y|, floor)
inline double max_rel_diff(const argument& x, const argument& y, double floor)
{
    auto a = x.to_vector<double>();
    auto b = y.to_vector<double>();
    if(a.size() != b.size())
        return INFINITY;
    double r = 0;
    for(std::size_t i = 0; i < a.size(); i++)
    {
        if(std::isnan(a[i]) != std::isnan(b[i]))
            return INFINITY;
        if(std::isnan(a[i]))
            continue;
        r = std::max(r, std::fabs(a[i] - b[i]) / std::max(std::fabs(b[i]), floor));
    }
    return r;
}

// quantizelinear / dequantizelinear with a scalar scale and zero point broadcast to x, the way
// the reference's tests add them (test/simplify_qdq_test.cpp:45-63)
inline instruction_ref add_quantize_op(module& m,
                                       const std::string& name,
                                       instruction_ref x,
                                       instruction_ref scale,
                                       instruction_ref shift)
{
    auto lens = x->get_shape().lens();
    auto s    = m.add_instruction(make_op("multibroadcast", {{"out_lens", lens}}), scale);
    auto z    = m.add_instruction(make_op("multibroadcast", {{"out_lens", lens}}), shift);
    return m.add_instruction(make_op(name), x, s, z);
}

inline instruction_ref
add_quantize_op(module& m, const std::string& name, instruction_ref x, instruction_ref scale)
{
    auto lens = x->get_shape().lens();
    auto s    = m.add_instruction(make_op("multibroadcast", {{"out_lens", lens}}), scale);
    return m.add_instruction(make_op(name), x, s);
}

} // namespace testutil
#endif
