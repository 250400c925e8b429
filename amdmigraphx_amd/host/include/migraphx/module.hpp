// An ordered list of instructions in SSA form (src/include/migraphx/module.hpp:61-340): every
// argument precedes its users; the module's results are the arguments of its `@return`, or its
// last instruction when there is none.
#ifndef MIGRAPHX_GUARD_MODULE_HPP
#define MIGRAPHX_GUARD_MODULE_HPP

#include <iosfwd>
#include <list>
#include <string>
#include <unordered_map>
#include <vector>
#include <migraphx/instruction.hpp>
#include <migraphx/register_op.hpp>

namespace migraphx {

struct module
{
    explicit module(std::string name = "main") : m_name(std::move(name)) {}
    module(const module& other);
    module& operator=(module other);
    module(module&&) noexcept = default;

    const std::string& name() const { return m_name; }

    template <class... Ts>
    instruction_ref add_instruction(const operation& op, Ts... args)
    {
        return insert_instruction(end(), op, std::vector<instruction_ref>{args...});
    }
    instruction_ref add_instruction(const operation& op, std::vector<instruction_ref> args)
    {
        return insert_instruction(end(), op, std::move(args));
    }
    template <class... Ts>
    instruction_ref insert_instruction(instruction_ref ins, const operation& op, Ts... args)
    {
        return insert_instruction(ins, op, std::vector<instruction_ref>{args...});
    }
    instruction_ref
    insert_instruction(instruction_ref ins, const operation& op, std::vector<instruction_ref> args);

    template <class... Ts>
    instruction_ref replace_instruction(instruction_ref ins, const operation& op, Ts... args)
    {
        return replace_instruction(ins, op, std::vector<instruction_ref>{args...});
    }
    instruction_ref
    replace_instruction(instruction_ref ins, const operation& op, std::vector<instruction_ref> args);
    // every user of ins uses rep instead
    instruction_ref replace_instruction(instruction_ref ins, instruction_ref rep);

    instruction_ref remove_instruction(instruction_ref ins);
    instruction_ref move_instruction(instruction_ref src, instruction_ref dst);

    instruction_ref add_literal(literal l) { return insert_literal(begin_after_literals(), std::move(l)); }
    template <class T>
    instruction_ref add_literal(const shape& s, const std::vector<T>& v)
    {
        return add_literal(literal{s, v});
    }
    instruction_ref insert_literal(instruction_ref ins, literal l);
    instruction_ref add_parameter(std::string name, shape s);
    // a parameter at a given position and rank among the parameters, as a saved program lists it
    instruction_ref
    insert_parameter(instruction_ref ins, std::string name, shape s, std::size_t order);
    instruction_ref add_return(std::vector<instruction_ref> args);

    std::vector<std::string> get_parameter_names() const;
    shape get_parameter_shape(const std::string& name) const;
    instruction_ref get_parameter(const std::string& name) const;
    std::unordered_map<std::string, shape> get_parameter_shapes() const;
    std::vector<shape> get_output_shapes() const;
    std::vector<instruction_ref> get_returns() const;

    bool has_instruction(instruction_ref ins) const;
    std::size_t size() const { return m_ins.size(); }
    instruction_ref begin() const { return const_cast<module*>(this)->m_ins.begin(); }
    instruction_ref end() const { return const_cast<module*>(this)->m_ins.end(); }

    // end() if the module is well formed, else the first offending instruction
    instruction_ref validate() const;
    void finalize(context& ctx);

    friend std::ostream& operator<<(std::ostream& os, const module& m);
    friend bool operator==(const module& x, const module& y);
    friend bool operator!=(const module& x, const module& y) { return not(x == y); }

    private:
    instruction_ref begin_after_literals() const { return begin(); }
    std::string m_name;
    std::list<instruction> m_ins;
};

// iterate instruction_refs of a module while it may be edited at the current position
struct iterator_for_module
{
    const module* m;
    struct iterator
    {
        instruction_ref it;
        instruction_ref operator*() const { return it; }
        iterator& operator++() { ++it; return *this; }
        bool operator!=(const iterator& o) const { return it != o.it; }
    };
    iterator begin() const { return {m->begin()}; }
    iterator end() const { return {m->end()}; }
};
inline iterator_for_module iterator_for(const module& m) { return {&m}; }

namespace builtin {
struct literal_op
{
    std::string name() const { return "@literal"; }
    shape compute_shape(const std::vector<shape>&) const { MIGRAPHX_THROW("builtin"); }
};
struct param
{
    std::string parameter;
    std::size_t order = 0;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.parameter, "parameter");
        f(self.order, "order");
    }
    std::string name() const { return "@param"; }
    shape compute_shape(const std::vector<shape>&) const { MIGRAPHX_THROW("builtin"); }
};
struct returns
{
    std::string name() const { return "@return"; }
    shape compute_shape(const std::vector<shape>&) const { return {}; }
};
} // namespace builtin

} // namespace migraphx
#endif
