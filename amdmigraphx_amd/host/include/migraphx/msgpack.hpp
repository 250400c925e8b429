// MessagePack form of a `value`, the default format of a saved program
// (src/include/migraphx/msgpack.hpp, mapping in src/msgpack.cpp:57-195): null -> nil, numbers in
// their shortest encoding, a list with keys -> map, any other list -> array, binary data -> an
// array of bin chunks of at most 2^32 - 2 bytes each.
#ifndef MIGRAPHX_GUARD_MSGPACK_HPP
#define MIGRAPHX_GUARD_MSGPACK_HPP

#include <cstddef>
#include <vector>
#include <migraphx/value.hpp>

namespace migraphx {

std::vector<char> to_msgpack(const value& v);
value from_msgpack(const char* buffer, std::size_t size);
value from_msgpack(const std::vector<char>& buffer);

} // namespace migraphx
#endif
