// One node of a module: operator, result shape, argument and user lists
// (src/include/migraphx/instruction.hpp).
#ifndef MIGRAPHX_GUARD_INSTRUCTION_HPP
#define MIGRAPHX_GUARD_INSTRUCTION_HPP

#include <list>
#include <string>
#include <vector>
#include <migraphx/argument.hpp>
#include <migraphx/operation.hpp>

namespace migraphx {

struct instruction;
using instruction_ref = std::list<instruction>::iterator;

struct instruction
{
    instruction() = default;
    instruction(operation o, shape r, std::vector<instruction_ref> args)
        : op(std::move(o)), result(std::move(r)), arguments(std::move(args))
    {
    }
    explicit instruction(literal l);

    std::string name() const { return op.name(); }
    const shape& get_shape() const { return result; }
    const operation& get_operator() const { return op; }
    operation& get_operator() { return op; }
    const std::vector<instruction_ref>& inputs() const { return arguments; }
    const std::vector<instruction_ref>& outputs() const { return output; }
    const literal& get_literal() const { return lit; }

    // true when the value is known at compile time: a literal, or a context-free operator whose
    // inputs all are
    bool can_eval() const;
    // the compile-time value, or an empty argument
    argument eval() const;

    // in `ins`, use `new_arg` wherever `old` is an argument; result shapes downstream are recomputed
    static void replace_argument(instruction_ref ins, instruction_ref old, instruction_ref new_arg);
    // recompute this instruction's shape and, if it changed, its users'
    static void recompute_shape(instruction_ref ins);

    void add_output(instruction_ref o);
    void remove_output(instruction_ref o);

    friend struct module;

    private:
    operation op;
    shape result;
    std::vector<instruction_ref> arguments;
    std::vector<instruction_ref> output;
    literal lit;
};

} // namespace migraphx

namespace std {
template <>
struct hash<migraphx::instruction_ref>
{
    size_t operator()(const migraphx::instruction_ref& x) const noexcept
    {
        return std::hash<const migraphx::instruction*>{}(&*x);
    }
};
} // namespace std
#endif
