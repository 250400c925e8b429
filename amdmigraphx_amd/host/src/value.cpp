#include <migraphx/value.hpp>
#include <algorithm>
#include <ostream>

namespace migraphx {

value::value(std::initializer_list<value> i)
{
    // {"key", x}: a key/value pair
    if(i.size() == 2 and i.begin()->is_string() and i.begin()->get_key().empty())
    {
        *this = *(i.begin() + 1);
        m_key = i.begin()->m_str;
        return;
    }
    m_items.assign(i.begin(), i.end());
    const bool all_keys = not m_items.empty() and
                          std::all_of(m_items.begin(), m_items.end(), [](const value& v) {
                              return not v.get_key().empty();
                          });
    m_kind = all_keys ? object_kind : array_kind;
}

bool value::contains(const std::string& key) const
{
    return std::any_of(
        m_items.begin(), m_items.end(), [&](const value& v) { return v.m_key == key; });
}

const value& value::at(const std::string& key) const
{
    auto it = std::find_if(
        m_items.begin(), m_items.end(), [&](const value& v) { return v.m_key == key; });
    if(it == m_items.end())
        MIGRAPHX_THROW("value: no key '" + key + "'");
    return *it;
}

value& value::operator[](const std::string& key)
{
    if(m_kind == null_kind)
        m_kind = object_kind;
    auto it = std::find_if(
        m_items.begin(), m_items.end(), [&](const value& v) { return v.m_key == key; });
    if(it != m_items.end())
        return *it;
    m_items.emplace_back();
    m_items.back().m_key = key;
    return m_items.back();
}

const value& value::at(std::size_t i) const
{
    if(i >= m_items.size())
        MIGRAPHX_THROW("value: index out of range");
    return m_items[i];
}

void value::push_back(const value& v)
{
    if(m_kind == null_kind)
        m_kind = v.get_key().empty() ? array_kind : object_kind;
    m_items.push_back(v);
}

void value::get(bool& b) const { b = as_int() != 0; }

const std::string& value::get_binary() const
{
    if(m_kind != binary_kind)
        MIGRAPHX_THROW("value: expected binary data");
    return m_str;
}

const std::string& value::get_string() const
{
    if(m_kind != string_kind)
        MIGRAPHX_THROW("value: expected a string");
    return m_str;
}

void value::get(std::string& s) const
{
    if(m_kind != string_kind)
        MIGRAPHX_THROW("value: expected a string");
    s = m_str;
}

int64_t value::as_int() const
{
    switch(m_kind)
    {
    case bool_kind:
    case int_kind: return m_int;
    case float_kind: return static_cast<int64_t>(m_float);
    case string_kind: return static_cast<int64_t>(shape::parse_type(m_str));
    default: MIGRAPHX_THROW("value: expected a number");
    }
}

double value::as_float() const
{
    switch(m_kind)
    {
    case bool_kind:
    case int_kind: return static_cast<double>(m_int);
    case float_kind: return m_float;
    default: MIGRAPHX_THROW("value: expected a number");
    }
}

bool operator==(const value& x, const value& y)
{
    if(x.m_key != y.m_key)
        return false;
    const bool xnum = x.m_kind == value::bool_kind or x.m_kind == value::int_kind or
                      x.m_kind == value::float_kind;
    const bool ynum = y.m_kind == value::bool_kind or y.m_kind == value::int_kind or
                      y.m_kind == value::float_kind;
    if(xnum and ynum)
        return x.as_float() == y.as_float();
    if(x.m_kind != y.m_kind)
        return false;
    if(x.m_kind == value::string_kind or x.m_kind == value::binary_kind)
        return x.m_str == y.m_str;
    return x.m_items == y.m_items;
}

std::ostream& operator<<(std::ostream& os, const value& v)
{
    switch(v.m_kind)
    {
    case value::null_kind: os << "null"; break;
    case value::bool_kind: os << (v.m_int != 0 ? "true" : "false"); break;
    case value::int_kind: os << v.m_int; break;
    case value::float_kind: os << v.m_float; break;
    case value::string_kind: os << v.m_str; break;
    case value::binary_kind: os << "binary[" << v.m_str.size() << "]"; break;
    case value::array_kind:
    case value::object_kind: {
        const bool obj = v.m_kind == value::object_kind;
        os << (obj ? "{" : "[");
        for(std::size_t i = 0; i < v.m_items.size(); i++)
        {
            if(i > 0)
                os << ", ";
            if(obj)
                os << v.m_items[i].m_key << ": ";
            os << v.m_items[i];
        }
        os << (obj ? "}" : "]");
        break;
    }
    }
    return os;
}

} // namespace migraphx
