// Target registry (src/include/migraphx/register_target.hpp:42-73, src/register_target.cpp:41-87).
// MIGRAPHX_REGISTER_TARGET(T) registers T{} while its shared library is loaded.  make_target(name)
// returns the registered target; when the name is unknown it first loads
// libmigraphx_<name>.so, whose static initialisers register the target and its operators.
#ifndef MIGRAPHX_GUARD_REGISTER_TARGET_HPP
#define MIGRAPHX_GUARD_REGISTER_TARGET_HPP

#include <string>
#include <vector>
#include <migraphx/target.hpp>

namespace migraphx {

void register_target(const target& t);
void unregister_target(const std::string& name);
target make_target(const std::string& name);
std::vector<std::string> get_targets();

template <class T>
struct target_handler
{
    std::string target_name;
    target_handler() : target_name(T{}.name()) { register_target(target{T{}}); }
    ~target_handler() { unregister_target(target_name); }
};

#define MIGRAPHX_REGISTER_TARGET(...) \
    static const migraphx::target_handler<__VA_ARGS__> migraphx_register_target_instance {}

} // namespace migraphx
#endif
