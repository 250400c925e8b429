#include <migraphx/program.hpp>
#include <migraphx/register_op.hpp>
#include <migraphx/register_target.hpp>
#include <migraphx/serialize.hpp>
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
    : m_main(std::make_unique<module>(*p.m_main)),
      m_ctx(p.m_ctx),
      m_target(p.m_target),
      m_compiled(p.m_compiled)
{
}

program& program::operator=(program p)
{
    std::swap(m_main, p.m_main);
    std::swap(m_ctx, p.m_ctx);
    std::swap(m_target, p.m_target);
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
    m_target   = t.name();
    m_compiled = true;
}

// --------------------------------------------------------------- saved programs

static const char* const library_version = "2.16.0";

value program::to_value() const
{
    value result                = value::object();
    result["version"]           = value("version", program_file_version);
    result["migraphx_version"]  = value("migraphx_version", library_version);
    value targets               = value::array();
    value contexts              = value::array();
    if(m_compiled)
    {
        value t   = value::object();
        t["name"] = value("name", m_target);
        targets.push_back(t);
        contexts.push_back(value::object()); // the stream is made anew on load
    }
    result["targets"]  = value("targets", targets);
    result["contexts"] = value("contexts", contexts);

    // results are named by position, parameters by their own name (src/module.cpp:1473-1500)
    std::unordered_map<const instruction*, std::string> names;
    value nodes       = value::array();
    std::size_t count = 0;
    for(auto ins = m_main->begin(); ins != m_main->end(); ++ins, ++count)
    {
        const bool is_param = ins->name() == "@param";
        const auto out      = is_param ? any_cast<builtin::param>(ins->get_operator()).parameter
                                       : "@" + std::to_string(count);
        names[&*ins]        = out;
        value node          = value::object();
        node["output"]      = value("output", out);
        node["name"]        = value("name", ins->name());
        node["shape"]       = value("shape", migraphx::to_value(ins->get_shape()));
        node["normalized"]  = value("normalized", true);
        if(ins->name() == "@literal")
            node["literal"] = value("literal", migraphx::to_value(ins->get_literal()));
        node["operator"] = value("operator", ins->get_operator().to_value());
        value inputs     = value::array();
        for(auto a : ins->inputs())
            inputs.push_back(value(names.at(&*a)));
        node["inputs"] = value("inputs", inputs);
        nodes.push_back(node);
    }
    value main_module     = value::object();
    main_module["name"]   = value("name", m_main->name());
    main_module["nodes"]  = value("nodes", nodes);
    value modules         = value::object();
    modules[m_main->name()] = value(m_main->name(), main_module);
    result["modules"]     = value("modules", modules);
    return result;
}

void program::from_value(const value& v)
{
    const auto version = v.at("version").to<int>();
    if(version != program_file_version)
        MIGRAPHX_THROW(
            "Error: Program version mismatch. MXR file was created using program file version: " +
            std::to_string(version) + ", while installed MIGraphX is using program file version: " +
            std::to_string(program_file_version) +
            ", Try regenerating MXR file using installed MIGraphX and running again.");
    const auto& targets = v.at("targets");
    if(targets.size() > 1)
        MIGRAPHX_THROW("from_value: programs compiled for several targets are not supported");
    const auto& modules = v.at("modules");
    if(modules.size() != 1 or not modules.contains("main"))
        MIGRAPHX_THROW("from_value: programs with submodules are not supported");

    // make_target loads the target's library, which registers its operators
    target tgt;
    if(not targets.empty())
        tgt = make_target(targets.at(0).at("name").to<std::string>());

    auto fresh = std::make_unique<module>("main");
    std::unordered_map<std::string, instruction_ref> by_name;
    for(const auto& node : modules.at("main").at("nodes").items())
    {
        const auto name    = node.at("name").to<std::string>();
        const auto& fields = node.at("operator");
        instruction_ref out;
        if(name == "@param")
        {
            out = fresh->insert_parameter(fresh->end(),
                                          fields.at("parameter").to<std::string>(),
                                          migraphx::from_value<shape>(node.at("shape")),
                                          fields.contains("order")
                                              ? fields.at("order").to<std::size_t>()
                                              : fresh->get_parameter_names().size());
        }
        else if(name == "@literal")
        {
            out = fresh->insert_literal(fresh->end(), migraphx::from_value<literal>(node.at("literal")));
        }
        else
        {
            std::vector<instruction_ref> inputs;
            for(const auto& i : node.at("inputs").items())
            {
                auto it = by_name.find(i.to<std::string>());
                if(it == by_name.end())
                    MIGRAPHX_THROW("from_value: " + name + " uses '" + i.to<std::string>() +
                                   "' before it is defined");
                inputs.push_back(it->second);
            }
            out = name == "@return" ? fresh->add_return(inputs)
                                    : fresh->add_instruction(make_op(name, fields), inputs);
        }
        by_name[node.at("output").to<std::string>()] = out;
    }

    m_main     = std::move(fresh);
    m_ctx      = context{};
    m_target   = "";
    m_compiled = false;
    if(not tgt.empty())
    {
        m_ctx = tgt.get_context();
        m_main->finalize(m_ctx);
        m_ctx.finish();
        m_target   = tgt.name();
        m_compiled = true;
    }
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
