#include <migraphx/module.hpp>
#include <algorithm>
#include <ostream>
#include <sstream>
#include <unordered_set>

namespace migraphx {

// ---------------------------------------------------------------- instruction

instruction::instruction(literal l)
    : op(builtin::literal_op{}), result(l.get_shape()), lit(std::move(l))
{
}

bool instruction::can_eval() const
{
    if(name() == "@literal")
        return true;
    if(name() == "@param" or name() == "@return")
        return false;
    if(not op.is_context_free())
        return false;
    return std::all_of(
        arguments.begin(), arguments.end(), [](instruction_ref i) { return i->can_eval(); });
}

argument instruction::eval() const
{
    if(name() == "@literal")
        return lit.get_argument();
    if(not can_eval())
        return {};
    std::vector<argument> args;
    for(auto i : arguments)
        args.push_back(i->eval());
    return op.compute(result, args);
}

void instruction::add_output(instruction_ref o)
{
    if(std::find(output.begin(), output.end(), o) == output.end())
        output.push_back(o);
}

void instruction::remove_output(instruction_ref o)
{
    output.erase(std::remove(output.begin(), output.end(), o), output.end());
}

void instruction::recompute_shape(instruction_ref ins)
{
    if(ins->name() == "@literal" or ins->name() == "@param" or ins->name() == "@return")
        return;
    std::vector<shape> in;
    for(auto a : ins->arguments)
        in.push_back(a->get_shape());
    shape r = ins->op.compute_shape(in);
    if(r == ins->result)
        return;
    ins->result = r;
    for(auto o : ins->output)
        recompute_shape(o);
}

void instruction::replace_argument(instruction_ref ins, instruction_ref old, instruction_ref new_arg)
{
    bool found = false;
    for(auto& a : ins->arguments)
    {
        if(a == old)
        {
            a     = new_arg;
            found = true;
        }
    }
    if(not found)
        return;
    old->remove_output(ins);
    new_arg->add_output(ins);
    recompute_shape(ins);
}

// --------------------------------------------------------------------- module

module::module(const module& other) : m_name(other.m_name)
{
    std::unordered_map<instruction_ref, instruction_ref> map;
    for(auto it = other.begin(); it != other.end(); ++it)
    {
        instruction copy = *it;
        copy.output.clear();
        for(auto& a : copy.arguments)
            a = map.at(a);
        m_ins.push_back(std::move(copy));
        auto n = std::prev(m_ins.end());
        for(auto a : n->arguments)
            a->add_output(n);
        map[it] = n;
    }
}

module& module::operator=(module other)
{
    std::swap(m_name, other.m_name);
    m_ins.swap(other.m_ins);
    return *this;
}

instruction_ref module::insert_instruction(instruction_ref ins,
                                           const operation& op,
                                           std::vector<instruction_ref> args)
{
    std::vector<shape> in;
    for(auto a : args)
        in.push_back(a->get_shape());
    shape r  = op.compute_shape(in);
    auto pos = m_ins.insert(ins, instruction{op, r, std::move(args)});
    for(auto a : pos->arguments)
        a->add_output(pos);
    return pos;
}

instruction_ref module::replace_instruction(instruction_ref ins,
                                            const operation& op,
                                            std::vector<instruction_ref> args)
{
    std::vector<shape> in;
    for(auto a : args)
        in.push_back(a->get_shape());
    shape r = op.compute_shape(in);
    for(auto a : ins->arguments)
        a->remove_output(ins);
    ins->op        = op;
    ins->arguments = std::move(args);
    ins->lit       = literal{};
    for(auto a : ins->arguments)
        a->add_output(ins);
    if(r != ins->result)
    {
        ins->result = r;
        for(auto o : ins->output)
            instruction::recompute_shape(o);
    }
    return ins;
}

instruction_ref module::replace_instruction(instruction_ref ins, instruction_ref rep)
{
    if(ins == rep)
        return ins;
    // a module without @return yields its last instruction: keep the replacement in that place
    if(ins == std::prev(end()) and ins->name() != "@return")
    {
        auto users = ins->output;
        for(auto o : users)
            instruction::replace_argument(o, ins, rep);
        remove_instruction(ins);
        move_instruction(rep, end());
        return rep;
    }
    auto users = ins->output;
    for(auto o : users)
        instruction::replace_argument(o, ins, rep);
    return rep;
}

instruction_ref module::remove_instruction(instruction_ref ins)
{
    if(not ins->output.empty())
        MIGRAPHX_THROW("remove_instruction: " + ins->name() + " still has users");
    for(auto a : ins->arguments)
        a->remove_output(ins);
    return m_ins.erase(ins);
}

instruction_ref module::move_instruction(instruction_ref src, instruction_ref dst)
{
    m_ins.splice(dst, m_ins, src);
    return src;
}

instruction_ref module::insert_literal(instruction_ref ins, literal l)
{
    return m_ins.insert(ins, instruction{std::move(l)});
}

instruction_ref module::add_parameter(std::string name, shape s)
{
    std::size_t order = get_parameter_names().size();
    m_ins.push_front(instruction{operation{builtin::param{std::move(name), order}}, std::move(s), {}});
    return m_ins.begin();
}

instruction_ref
module::insert_parameter(instruction_ref ins, std::string name, shape s, std::size_t order)
{
    return m_ins.insert(
        ins, instruction{operation{builtin::param{std::move(name), order}}, std::move(s), {}});
}

instruction_ref module::add_return(std::vector<instruction_ref> args)
{
    m_ins.push_back(instruction{operation{builtin::returns{}}, shape{}, std::move(args)});
    auto r = std::prev(m_ins.end());
    for(auto a : r->arguments)
        a->add_output(r);
    return r;
}

std::vector<std::string> module::get_parameter_names() const
{
    std::vector<std::pair<std::size_t, std::string>> ps;
    for(const auto& i : m_ins)
    {
        if(i.name() == "@param")
        {
            const auto& p = any_cast<builtin::param>(i.get_operator());
            ps.emplace_back(p.order, p.parameter);
        }
    }
    std::sort(ps.begin(), ps.end());
    std::vector<std::string> r;
    for(auto& p : ps)
        r.push_back(p.second);
    return r;
}

instruction_ref module::get_parameter(const std::string& name) const
{
    for(auto it = begin(); it != end(); ++it)
    {
        if(it->name() == "@param" and any_cast<builtin::param>(it->get_operator()).parameter == name)
            return it;
    }
    return end();
}

shape module::get_parameter_shape(const std::string& name) const
{
    auto it = get_parameter(name);
    if(it == end())
        return {};
    return it->get_shape();
}

std::unordered_map<std::string, shape> module::get_parameter_shapes() const
{
    std::unordered_map<std::string, shape> r;
    for(const auto& n : get_parameter_names())
        r[n] = get_parameter_shape(n);
    return r;
}

std::vector<instruction_ref> module::get_returns() const
{
    if(m_ins.empty())
        return {};
    auto last = std::prev(end());
    if(last->name() == "@return")
        return last->inputs();
    return {last};
}

std::vector<shape> module::get_output_shapes() const
{
    std::vector<shape> r;
    for(auto i : get_returns())
        r.push_back(i->get_shape());
    return r;
}

bool module::has_instruction(instruction_ref ins) const
{
    for(auto it = begin(); it != end(); ++it)
    {
        if(it == ins)
            return true;
    }
    return false;
}

instruction_ref module::validate() const
{
    std::unordered_set<const instruction*> seen;
    for(auto it = begin(); it != end(); ++it)
    {
        for(auto a : it->inputs())
        {
            if(seen.count(&*a) == 0)
                return it;
        }
        seen.insert(&*it);
    }
    return end();
}

void module::finalize(context& ctx)
{
    for(auto it = begin(); it != end(); ++it)
    {
        if(it->name()[0] == '@')
            continue;
        std::vector<shape> in;
        for(auto a : it->inputs())
            in.push_back(a->get_shape());
        it->op.finalize(ctx, it->get_shape(), in);
    }
}

std::ostream& operator<<(std::ostream& os, const module& m)
{
    std::unordered_map<const instruction*, std::string> names;
    std::size_t count = 0;
    for(auto it = m.begin(); it != m.end(); ++it)
    {
        std::string n;
        if(it->name() == "@param")
            n = any_cast<builtin::param>(it->get_operator()).parameter;
        else
            n = "@" + std::to_string(count++);
        names[&*it] = n;
        os << n << " = ";
        if(it->name() == "@literal")
            os << "@literal{" << it->get_literal() << "}";
        else if(it->name() == "@param")
            os << "@param:" << n;
        else
            os << it->get_operator();
        if(not it->inputs().empty())
        {
            os << "(";
            for(std::size_t i = 0; i < it->inputs().size(); i++)
                os << (i == 0 ? "" : ",") << names[&*it->inputs()[i]];
            os << ")";
        }
        os << " -> " << it->get_shape() << "\n";
    }
    return os;
}

bool operator==(const module& x, const module& y)
{
    std::stringstream a;
    std::stringstream b;
    a << x;
    b << y;
    return a.str() == b.str();
}

} // namespace migraphx
