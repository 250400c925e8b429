// Conversions between IR types and `value`, the form a saved program is made of.  The layouts
// follow the reference so that its files describe the same fields: a shape is
// {type, sub_shapes, lens, strides, dynamic_dimensions, dyn_strides} (src/shape.cpp:1403-1429), a
// literal or host argument is {shape, data} with the bytes in memory order
// (src/serialize.cpp:33-69).
#ifndef MIGRAPHX_GUARD_SERIALIZE_HPP
#define MIGRAPHX_GUARD_SERIALIZE_HPP

#include <string>
#include <type_traits>
#include <vector>
#include <migraphx/argument.hpp>
#include <migraphx/value.hpp>

namespace migraphx {

value to_value(const shape& s);
value to_value(const literal& l);
// host memory only: a target copies its buffers back before it converts them
value to_value(const argument& a);
template <class T>
value to_value(const std::vector<T>& v);
template <class T, std::enable_if_t<std::is_constructible<value, const T&>{}, int> = 0>
value to_value(const T& x)
{
    return value(x);
}
template <class T>
value to_value(const std::vector<T>& v)
{
    value r = value::array();
    for(const auto& x : v)
        r.push_back(to_value(x));
    return r;
}

void from_value(const value& v, shape& s);
void from_value(const value& v, literal& l);
void from_value(const value& v, argument& a);
template <class T>
void from_value(const value& v, std::vector<T>& out);
template <class T, std::enable_if_t<std::is_constructible<value, const T&>{}, int> = 0>
void from_value(const value& v, T& x)
{
    v.get(x);
}
template <class T>
void from_value(const value& v, std::vector<T>& out)
{
    if(not v.is_array() and not v.is_object() and not v.is_null())
        MIGRAPHX_THROW("from_value: expected an array");
    out.clear();
    for(const auto& item : v.items())
    {
        T x{};
        from_value(item, x);
        out.push_back(std::move(x));
    }
}
template <class T>
T from_value(const value& v)
{
    T x{};
    from_value(v, x);
    return x;
}

} // namespace migraphx
#endif
