#include <migraphx/program.hpp>
#include <migraphx/register_op.hpp>
#include <migraphx/register_target.hpp>
#include <algorithm>
#include <iostream>
#include <map>
#include <mutex>
#include <ostream>
#include <dlfcn.h>

namespace migraphx {

// ------------------------------------------------------------------ registries
// Written at static initialisation (and when a target library is loaded), read afterwards; the
// lock makes loading a target library from concurrent threads safe.

namespace {
std::mutex& registry_mutex()
{
    static std::mutex m;
    return m;
}
std::map<std::string, operation>& op_map()
{
    static std::map<std::string, operation> m;
    return m;
}
std::map<std::string, target>& target_map()
{
    static std::map<std::string, target> m;
    return m;
}
} // namespace

void register_op(const operation& op)
{
    std::lock_guard<std::mutex> lock(registry_mutex());
    op_map()[op.name()] = op;
}
void unregister_op(const std::string& name)
{
    std::lock_guard<std::mutex> lock(registry_mutex());
    op_map().erase(name);
}
bool has_op(const std::string& name)
{
    std::lock_guard<std::mutex> lock(registry_mutex());
    return op_map().count(name) > 0;
}
operation load_op(const std::string& name)
{
    std::lock_guard<std::mutex> lock(registry_mutex());
    auto it = op_map().find(name);
    if(it == op_map().end())
        MIGRAPHX_THROW("Operator not found: " + name);
    return it->second;
}
std::vector<std::string> get_operators()
{
    std::lock_guard<std::mutex> lock(registry_mutex());
    std::vector<std::string> r;
    for(auto& p : op_map())
        r.push_back(p.first);
    return r;
}
operation make_op(const std::string& name) { return load_op(name); }
operation make_op(const std::string& name, const value& v)
{
    auto op = load_op(name);
    if(not v.is_object() and not v.is_null() and not v.empty())
        MIGRAPHX_THROW("make_op: attributes of " + name + " must be key/value pairs");
    // reject unknown attribute names, as the reference's from_value does
    auto known = op.to_value();
    for(const auto& item : v.items())
    {
        if(not known.contains(item.get_key()))
            MIGRAPHX_THROW("make_op: " + name + " has no attribute '" + item.get_key() + "'");
    }
    op.from_value(v);
    return op;
}

void register_target(const target& t)
{
    std::lock_guard<std::mutex> lock(registry_mutex());
    target_map()[t.name()] = t;
}
void unregister_target(const std::string& name)
{
    std::lock_guard<std::mutex> lock(registry_mutex());
    target_map().erase(name);
}
std::vector<std::string> get_targets()
{
    std::lock_guard<std::mutex> lock(registry_mutex());
    std::vector<std::string> r;
    for(auto& p : target_map())
        r.push_back(p.first);
    return r;
}

static bool target_known(const std::string& name)
{
    std::lock_guard<std::mutex> lock(registry_mutex());
    return target_map().count(name) > 0;
}

target make_target(const std::string& name)
{
    if(not target_known(name))
    {
        // the library stays loaded for the life of the process
        const std::string lib = "libmigraphx_" + name + ".so";
        void* h               = dlopen(lib.c_str(), RTLD_GLOBAL | RTLD_NOW);
        if(h == nullptr)
        {
            // next to this library
            Dl_info info{};
            if(dladdr(reinterpret_cast<void*>(&target_known), &info) != 0 and info.dli_fname != nullptr)
            {
                std::string dir = info.dli_fname;
                auto slash      = dir.find_last_of('/');
                dir             = slash == std::string::npos ? "." : dir.substr(0, slash);
                h               = dlopen((dir + "/" + lib).c_str(), RTLD_GLOBAL | RTLD_NOW);
            }
        }
        if(h == nullptr)
        {
            const char* err = dlerror();
            MIGRAPHX_THROW("Requested target '" + name + "' is not loaded or not supported (" +
                           std::string(err != nullptr ? err : lib.c_str()) + ")");
        }
    }
    std::lock_guard<std::mutex> lock(registry_mutex());
    auto it = target_map().find(name);
    if(it == target_map().end())
        MIGRAPHX_THROW("Requested target '" + name + "' is not loaded or not supported");
    return it->second;
}

// ---------------------------------------------------------------------- passes

void run_passes(module& m, const std::vector<pass>& passes)
{
    for(const auto& p : passes)
    {
        p.apply(m);
        auto bad = m.validate();
        if(bad != m.end())
            MIGRAPHX_THROW(p.name() + " pass produces invalid program at instruction " + bad->name());
    }
}

void run_passes(program& p, const std::vector<pass>& passes)
{
    run_passes(*p.get_main_module(), passes);
}

// --------------------------------------------------------------------- program

program::program(const program& p)
    : m_main(std::make_unique<module>(*p.m_main)), m_ctx(p.m_ctx), m_compiled(p.m_compiled)
{
}

program& program::operator=(program p)
{
    std::swap(m_main, p.m_main);
    std::swap(m_ctx, p.m_ctx);
    std::swap(m_compiled, p.m_compiled);
    return *this;
}

void program::compile(const target& t, compile_options options)
{
    if(m_compiled)
        MIGRAPHX_THROW("program is already compiled");
    m_ctx = t.get_context();
    run_passes(*this, t.get_passes(m_ctx, options));
    auto bad = m_main->validate();
    if(bad != m_main->end())
        MIGRAPHX_THROW("Invalid program from compilation at instruction " + bad->name());
    m_main->finalize(m_ctx);
    m_ctx.finish();
    m_compiled = true;
}

std::vector<argument> program::eval(const parameter_map& params) const
{
    std::unordered_map<const instruction*, argument> results;
    results.reserve(m_main->size());
    std::vector<argument> out;
    const instruction* last = nullptr;
    for(auto it = m_main->begin(); it != m_main->end(); ++it)
    {
        const auto& name = it->name();
        last             = &*it;
        if(name == "@literal")
        {
            results[&*it] = it->get_literal().get_argument();
        }
        else if(name == "@param")
        {
            const auto& pname = any_cast<builtin::param>(it->get_operator()).parameter;
            auto p            = params.find(pname);
            if(p == params.end())
                MIGRAPHX_THROW("Parameter not found: " + pname);
            if(p->second.get_shape() != it->get_shape())
                MIGRAPHX_THROW("Incorrect shape for parameter " + pname);
            results[&*it] = p->second;
        }
        else if(name == "@return")
        {
            for(auto a : it->inputs())
                out.push_back(results.at(&*a));
            return out;
        }
        else
        {
            std::vector<argument> args;
            args.reserve(it->inputs().size());
            for(auto a : it->inputs())
                args.push_back(results.at(&*a));
            results[&*it] = it->get_operator().compute(m_ctx, it->get_shape(), args);
        }
    }
    if(last != nullptr)
        out.push_back(results.at(last));
    return out;
}

std::ostream& operator<<(std::ostream& os, const program& p) { return os << *p.m_main; }

} // namespace migraphx
