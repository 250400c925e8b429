// JSON text form of a `value` (src/include/migraphx/json.hpp; src/json.cpp:58-160): objects keep
// their key order, binary data is written as {"bytes": [b0, b1, ...]} and read back from an
// object whose only member is "bytes".
#ifndef MIGRAPHX_GUARD_JSON_HPP
#define MIGRAPHX_GUARD_JSON_HPP

#include <cstddef>
#include <string>
#include <migraphx/value.hpp>

namespace migraphx {

std::string to_json_string(const value& v);
value from_json_string(const char* text, std::size_t size);
value from_json_string(const std::string& text);

} // namespace migraphx
#endif
