// A program owns its main module, and after compile() the target's context
// (src/include/migraphx/program.hpp; compile src/program.cpp:322-355, eval :549-558).
#ifndef MIGRAPHX_GUARD_PROGRAM_HPP
#define MIGRAPHX_GUARD_PROGRAM_HPP

#include <iosfwd>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>
#include <migraphx/module.hpp>
#include <migraphx/target.hpp>

namespace migraphx {

using parameter_map = std::unordered_map<std::string, argument>;

struct program
{
    program() : m_main(std::make_unique<module>("main")) {}
    program(const program& p);
    program& operator=(program p);
    program(program&&) noexcept = default;

    module* get_main_module() { return m_main.get(); }
    const module* get_main_module() const { return m_main.get(); }

    std::vector<std::string> get_parameter_names() const { return m_main->get_parameter_names(); }
    shape get_parameter_shape(const std::string& n) const { return m_main->get_parameter_shape(n); }
    std::unordered_map<std::string, shape> get_parameter_shapes() const
    {
        return m_main->get_parameter_shapes();
    }
    std::vector<shape> get_output_shapes() const { return m_main->get_output_shapes(); }

    // lower the program with the target's passes, then finalize every operator
    void compile(const target& t, compile_options options = compile_options{});
    bool is_compiled() const { return m_compiled; }
    // run the instructions in order on the calling thread; device work is asynchronous on the
    // context's stream until finish()
    std::vector<argument> eval(const parameter_map& params) const;
    void finish() const { m_ctx.finish(); }
    context& get_context() { return m_ctx; }

    // The saved form (src/program.cpp:720-777): version numbers, the target's name and context
    // when compiled, and per module the instructions in order, each with the name of its
    // result, operator fields, literal data and the names of its inputs.
    value to_value() const;
    // Rebuild from the saved form; a compiled program loads its target's library, takes a new
    // context from it and finalizes again (src/program.cpp:851-902).
    void from_value(const value& v);
    static constexpr int program_file_version = 8;

    friend std::ostream& operator<<(std::ostream& os, const program& p);
    friend bool operator==(const program& x, const program& y) { return *x.m_main == *y.m_main; }
    friend bool operator!=(const program& x, const program& y) { return not(x == y); }

    private:
    std::unique_ptr<module> m_main;
    mutable context m_ctx;
    std::string m_target; // name of the target it was compiled for
    bool m_compiled = false;
};

} // namespace migraphx
#endif
