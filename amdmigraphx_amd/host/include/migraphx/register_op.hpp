// Operator registry: name -> default-constructed operation
// (src/include/migraphx/register_op.hpp:60-80).  MIGRAPHX_REGISTER_OP(T) registers at static
// initialisation; make_op(name, attributes) copies the prototype and applies from_value.
#ifndef MIGRAPHX_GUARD_REGISTER_OP_HPP
#define MIGRAPHX_GUARD_REGISTER_OP_HPP

#include <string>
#include <vector>
#include <migraphx/operation.hpp>

namespace migraphx {

void register_op(const operation& op);
void unregister_op(const std::string& name);
bool has_op(const std::string& name);
operation load_op(const std::string& name);
std::vector<std::string> get_operators();

template <class T>
struct register_op_action
{
    register_op_action() { register_op(operation{T{}}); }
};

operation make_op(const std::string& name);
operation make_op(const std::string& name, const value& v);

#define MIGRAPHX_REGISTER_OP_CAT2(a, b) a##b
#define MIGRAPHX_REGISTER_OP_CAT(a, b) MIGRAPHX_REGISTER_OP_CAT2(a, b)
#define MIGRAPHX_REGISTER_OP(...)                                      \
    static const migraphx::register_op_action<__VA_ARGS__> MIGRAPHX_REGISTER_OP_CAT( \
        migraphx_register_op_, __LINE__) {}

} // namespace migraphx
#endif
