// Exceptions of the host layer: one exception type carrying "file:line: function: message",
// raised through MIGRAPHX_THROW (the convention of src/include/migraphx/errors.hpp:36-81).
#ifndef MIGRAPHX_GUARD_ERRORS_HPP
#define MIGRAPHX_GUARD_ERRORS_HPP

#include <stdexcept>
#include <string>

namespace migraphx {

struct exception : std::runtime_error
{
    unsigned int error;
    explicit exception(unsigned int e = 0, const std::string& msg = "")
        : std::runtime_error(msg), error(e)
    {
    }
};

inline exception
make_exception(const char* file, int line, const char* func, const std::string& msg)
{
    return exception(0, std::string(file) + ":" + std::to_string(line) + ": " + func + ": " + msg);
}

} // namespace migraphx

#define MIGRAPHX_THROW(...) \
    throw migraphx::make_exception(__FILE__, __LINE__, __func__, std::string(__VA_ARGS__))

#endif
