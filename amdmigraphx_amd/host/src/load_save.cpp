#include <migraphx/load_save.hpp>
#include <migraphx/json.hpp>
#include <migraphx/msgpack.hpp>
#include <fstream>

namespace migraphx {

program load_buffer(const char* buffer, std::size_t size, const file_options& options)
{
    value v;
    if(options.format == "msgpack")
        v = from_msgpack(buffer, size);
    else if(options.format == "json")
        v = from_json_string(buffer, size);
    else
        MIGRAPHX_THROW("Unknown format: " + options.format);
    program p;
    p.from_value(v);
    return p;
}

program load_buffer(const std::vector<char>& buffer, const file_options& options)
{
    return load_buffer(buffer.data(), buffer.size(), options);
}

program load(const std::string& filename, const file_options& options)
{
    std::ifstream is(filename, std::ios::binary | std::ios::ate);
    if(not is)
        MIGRAPHX_THROW("Failure opening file: " + filename);
    const auto size = static_cast<std::size_t>(is.tellg());
    if(size == 0)
        MIGRAPHX_THROW("Invalid size for: " + filename);
    std::vector<char> buffer(size);
    is.seekg(0);
    if(not is.read(buffer.data(), static_cast<std::streamsize>(size)))
        MIGRAPHX_THROW("Error reading file: " + filename);
    return load_buffer(buffer, options);
}

std::vector<char> save_buffer(const program& p, const file_options& options)
{
    const auto v = p.to_value();
    if(options.format == "msgpack")
        return to_msgpack(v);
    if(options.format == "json")
    {
        const auto text = to_json_string(v);
        return {text.begin(), text.end()};
    }
    MIGRAPHX_THROW("Unknown format: " + options.format);
}

void save(const program& p, const std::string& filename, const file_options& options)
{
    const auto buffer = save_buffer(p, options);
    std::ofstream os(filename, std::ios::binary);
    if(not os.write(buffer.data(), static_cast<std::streamsize>(buffer.size())))
        MIGRAPHX_THROW("Failure writing file: " + filename);
}

} // namespace migraphx
