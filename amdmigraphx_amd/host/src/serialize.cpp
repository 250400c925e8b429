#include <migraphx/serialize.hpp>

namespace migraphx {

value to_value(const shape& s)
{
    value r            = value::object();
    r["type"]          = value("type", s.type_string());
    r["sub_shapes"]    = value("sub_shapes", value::array());
    r["lens"]          = value("lens", s.lens());
    r["strides"]       = value("strides", s.strides());
    r["dynamic_dimensions"] = value("dynamic_dimensions", value::array());
    r["dyn_strides"]   = value("dyn_strides", value::array());
    return r;
}

void from_value(const value& v, shape& s)
{
    const auto type = v.at("type").get_string();
    if(type == "tuple_type")
        MIGRAPHX_THROW("from_value: tuple shapes are not supported");
    if(v.contains("dynamic_dimensions") and not v.at("dynamic_dimensions").empty())
        MIGRAPHX_THROW("from_value: dynamic shapes are not supported");
    s = shape{shape::parse_type(type),
              v.at("lens").to_vector<std::size_t>(),
              v.at("strides").to_vector<std::size_t>()};
}

static value raw_to_value(const shape& s, const char* bytes)
{
    value r    = value::object();
    r["shape"] = value("shape", to_value(s));
    if(bytes != nullptr)
        r["data"] = value("data", value::binary(bytes, s.bytes()));
    return r;
}

value to_value(const literal& l) { return raw_to_value(l.get_shape(), l.empty() ? nullptr : l.data()); }
value to_value(const argument& a) { return raw_to_value(a.get_shape(), a.empty() ? nullptr : a.data()); }

void from_value(const value& v, literal& l)
{
    shape s;
    from_value(v.at("shape"), s);
    if(not v.contains("data"))
    {
        l = literal{};
        return;
    }
    const auto& bytes = v.at("data").get_binary();
    if(bytes.size() != s.bytes())
        MIGRAPHX_THROW("from_value: literal of " + std::to_string(s.bytes()) + " bytes carries " +
                       std::to_string(bytes.size()));
    l = literal{s, bytes.data()};
}

void from_value(const value& v, argument& a)
{
    literal l;
    from_value(v, l);
    a = l.get_argument();
}

} // namespace migraphx
