#include <migraphx/load_save.hpp>
#include <migraphx/json.hpp>
#include <migraphx/msgpack.hpp>
#include <migraphx/serialize.hpp>
#include <fstream>
#include <type_traits>

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

static std::vector<char> read_file(const std::string& filename)
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
    return buffer;
}

static void write_file(const std::string& filename, const std::vector<char>& buffer)
{
    std::ofstream os(filename, std::ios::binary);
    if(not os.write(buffer.data(), static_cast<std::streamsize>(buffer.size())))
        MIGRAPHX_THROW("Failure writing file: " + filename);
}

program load(const std::string& filename, const file_options& options)
{
    return load_buffer(read_file(filename), options);
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
    write_file(filename, save_buffer(p, options));
}

void save_argument(const argument& a, const std::string& filename)
{
    write_file(filename, to_msgpack(to_value(a)));
}

argument load_argument(const std::string& filename)
{
    return from_value<argument>(from_msgpack(read_file(filename)));
}

argument generate_argument(const shape& s, unsigned long seed)
{
    argument result{s};
    unsigned long x = 123456789;
    unsigned long y = 362436069;
    unsigned long z = 521288629ULL ^ seed;
    auto next       = [&] {
        x ^= x << 16U;
        x ^= x >> 5U;
        x ^= x << 1U;
        const unsigned long t = x;
        x                     = y;
        y                     = z;
        z                     = t ^ x ^ y;
        return z;
    };
    const std::size_t n = s.element_space();
    if(s.type() == shape::fp4x2_type or s.type() == shape::tuple_type)
    {
        // bytes, drawn like uint8 (generate.cpp:90-96)
        auto* p = reinterpret_cast<unsigned char*>(result.data());
        for(std::size_t i = 0; i < n; i++)
            p[i] = static_cast<unsigned char>(next() % 32);
        return result;
    }
    visit_type(s.type(), [&](auto tag) {
        using T = decltype(tag);
        auto* p = reinterpret_cast<T*>(result.data());
        for(std::size_t i = 0; i < n; i++)
        {
            const unsigned long r = next();
            if constexpr(std::is_same<T, bool>{})
                p[i] = (r % 2) != 0;
            else if constexpr(std::is_integral<T>{} and std::is_unsigned<T>{})
                p[i] = static_cast<T>(r % (1ULL << (sizeof(T) * 5)));
            else if constexpr(std::is_integral<T>{})
            {
                const long long max = 1LL << (sizeof(T) * 5);
                p[i] = static_cast<T>(max / 2 - static_cast<long long>(r % static_cast<unsigned long>(max)));
            }
            else
                p[i] = T(static_cast<float>(-1.0 + static_cast<double>(r % 32) / 16.0));
        }
    });
    return result;
}

} // namespace migraphx
