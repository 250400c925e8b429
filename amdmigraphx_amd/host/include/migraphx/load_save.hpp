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

// one host argument as a MessagePack file (src/argument.cpp:219-227)
void save_argument(const argument& a, const std::string& filename);
argument load_argument(const std::string& filename);

// Repeatable test data (src/include/migraphx/generate.hpp:42-113, the default `legacy` mode): a
// xorshf96 sequence seeded with 521288629 ^ seed; floating types take -1 + (z mod 32) / 16, signed
// integers 2^(5 bytes - 1) - z mod 2^(5 bytes), unsigned integers z mod 2^(5 bytes), bool z mod 2.
argument generate_argument(const shape& s, unsigned long seed = 0);

} // namespace migraphx
#endif
