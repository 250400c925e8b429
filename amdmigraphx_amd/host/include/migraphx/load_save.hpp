// Programs on disk (src/include/migraphx/load_save.hpp:33-52): the `.mxr` file is the program's
// saved form in MessagePack ("msgpack", the default) or JSON ("json").
#ifndef MIGRAPHX_GUARD_LOAD_SAVE_HPP
#define MIGRAPHX_GUARD_LOAD_SAVE_HPP

#include <string>
#include <vector>
#include <migraphx/program.hpp>

namespace migraphx {

struct file_options
{
    std::string format = "msgpack";
};

program load(const std::string& filename, const file_options& options = file_options{});
program load_buffer(const std::vector<char>& buffer, const file_options& options = file_options{});
program load_buffer(const char* buffer, std::size_t size, const file_options& options = file_options{});

void save(const program& p, const std::string& filename, const file_options& options = file_options{});
std::vector<char> save_buffer(const program& p, const file_options& options = file_options{});

} // namespace migraphx
#endif
