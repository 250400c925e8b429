#include <migraphx/shape.hpp>
#include <algorithm>
#include <functional>
#include <numeric>
#include <ostream>

namespace migraphx {

shape::shape(type_t t, std::vector<std::size_t> l) : m_type(t), m_lens(std::move(l))
{
    calculate_strides();
}

shape::shape(type_t t, std::vector<std::size_t> l, std::vector<std::size_t> s)
    : m_type(t), m_lens(std::move(l)), m_strides(std::move(s))
{
    if(m_lens.size() != m_strides.size())
        MIGRAPHX_THROW("shape: lens and strides differ in rank");
}

void shape::calculate_strides()
{
    m_strides.assign(m_lens.size(), 1);
    for(std::size_t i = m_lens.size(); i > 1; i--)
        m_strides[i - 2] = m_strides[i - 1] * m_lens[i - 1];
}

shape shape::from_permutation(type_t t,
                              const std::vector<std::size_t>& l,
                              const std::vector<int64_t>& perm)
{
    if(perm.size() != l.size())
        MIGRAPHX_THROW("from_permutation: rank mismatch");
    // memory order: dimension perm[0] outermost ... perm[n-1] innermost
    std::vector<std::size_t> strides(l.size(), 1);
    std::size_t run = 1;
    for(std::size_t i = perm.size(); i > 0; i--)
    {
        strides[perm[i - 1]] = run;
        run *= l[perm[i - 1]];
    }
    return {t, l, strides};
}

std::size_t shape::elements() const
{
    if(m_lens.empty())
        return 0;
    return std::accumulate(m_lens.begin(), m_lens.end(), std::size_t{1}, std::multiplies<>{});
}

std::size_t shape::type_size(type_t t)
{
    switch(t)
    {
    case bool_type:
    case uint8_type:
    case int8_type:
    case fp8e4m3fnuz_type:
    case fp8e4m3fn_type:
    case fp8e5m2_type:
    case fp8e5m2fnuz_type:
    case fp4x2_type: return 1;
    case half_type:
    case bf16_type:
    case uint16_type:
    case int16_type: return 2;
    case float_type:
    case int32_type:
    case uint32_type: return 4;
    case double_type:
    case int64_type:
    case uint64_type: return 8;
    default: return 0;
    }
}

std::size_t shape::element_space() const
{
    if(m_lens.empty())
        return 0;
    if(std::any_of(m_lens.begin(), m_lens.end(), [](auto l) { return l == 0; }))
        return 0;
    std::size_t last = 0;
    for(std::size_t i = 0; i < m_lens.size(); i++)
        last += (m_lens[i] - 1) * m_strides[i];
    return last + 1;
}

std::size_t shape::index(const std::vector<std::size_t>& multi) const
{
    if(multi.size() != m_lens.size())
        MIGRAPHX_THROW("shape::index: rank mismatch");
    std::size_t r = 0;
    for(std::size_t i = 0; i < multi.size(); i++)
        r += multi[i] * m_strides[i];
    return r;
}

std::size_t shape::index(std::size_t i) const
{
    if(standard())
        return i;
    std::size_t r = 0;
    for(std::size_t d = m_lens.size(); d > 0; d--)
    {
        r += (i % m_lens[d - 1]) * m_strides[d - 1];
        i /= m_lens[d - 1];
    }
    return r;
}

std::vector<std::size_t> shape::multi(std::size_t i) const
{
    std::vector<std::size_t> r(m_lens.size());
    for(std::size_t d = m_lens.size(); d > 0; d--)
    {
        r[d - 1] = i % m_lens[d - 1];
        i /= m_lens[d - 1];
    }
    return r;
}

bool shape::packed() const { return not m_lens.empty() and elements() == element_space(); }

bool shape::transposed() const
{
    if(broadcasted())
    {
        // ignore the broadcast dimensions
        std::vector<std::size_t> s;
        std::copy_if(m_strides.begin(), m_strides.end(), std::back_inserter(s), [](auto x) {
            return x != 0;
        });
        return not std::is_sorted(s.rbegin(), s.rend());
    }
    return not std::is_sorted(m_strides.rbegin(), m_strides.rend());
}

bool shape::broadcasted() const
{
    return std::any_of(m_strides.begin(), m_strides.end(), [](auto s) { return s == 0; });
}

bool shape::scalar() const
{
    return not m_lens.empty() and
           std::all_of(m_strides.begin(), m_strides.end(), [](auto s) { return s == 0; });
}

bool shape::standard() const
{
    if(m_lens.empty())
        return false;
    std::size_t run = 1;
    for(std::size_t i = m_lens.size(); i > 0; i--)
    {
        // a dimension of length 1 may carry any stride
        if(m_lens[i - 1] != 1 and m_strides[i - 1] != run)
            return false;
        run *= m_lens[i - 1];
    }
    return true;
}

shape shape::normalize_standard() const
{
    if(standard())
        return {m_type, m_lens};
    return *this;
}

shape shape::with_lens(type_t t, const std::vector<std::size_t>& l) const
{
    if(l.size() != m_lens.size())
        MIGRAPHX_THROW("with_lens: rank mismatch");
    // keep the memory order of this shape
    std::vector<int64_t> perm(l.size());
    std::iota(perm.begin(), perm.end(), 0);
    std::stable_sort(perm.begin(), perm.end(), [&](auto a, auto b) {
        return m_strides[a] > m_strides[b];
    });
    return from_permutation(t, l, perm);
}

shape shape::with_type(type_t t) const
{
    shape r  = *this;
    r.m_type = t;
    return r;
}

std::string shape::type_name(type_t t)
{
    switch(t)
    {
    case bool_type: return "bool_type";
    case half_type: return "half_type";
    case float_type: return "float_type";
    case double_type: return "double_type";
    case uint8_type: return "uint8_type";
    case int8_type: return "int8_type";
    case uint16_type: return "uint16_type";
    case int16_type: return "int16_type";
    case int32_type: return "int32_type";
    case int64_type: return "int64_type";
    case uint32_type: return "uint32_type";
    case uint64_type: return "uint64_type";
    case fp8e4m3fnuz_type: return "fp8e4m3fnuz_type";
    case fp8e4m3fn_type: return "fp8e4m3fn_type";
    case fp8e5m2_type: return "fp8e5m2_type";
    case bf16_type: return "bf16_type";
    case fp8e5m2fnuz_type: return "fp8e5m2fnuz_type";
    case tuple_type: return "tuple_type";
    case fp4x2_type: return "fp4x2_type";
    }
    return "unknown_type";
}

shape::type_t shape::parse_type(const std::string& s)
{
    for(int i = 0; i <= fp4x2_type; i++)
    {
        auto n = type_name(static_cast<type_t>(i));
        if(s == n or s + "_type" == n)
            return static_cast<type_t>(i);
    }
    MIGRAPHX_THROW("Unknown type: " + s);
}

bool shape::is_integral(type_t t)
{
    switch(t)
    {
    case bool_type:
    case uint8_type:
    case int8_type:
    case uint16_type:
    case int16_type:
    case int32_type:
    case int64_type:
    case uint32_type:
    case uint64_type: return true;
    default: return false;
    }
}

bool shape::is_unsigned(type_t t)
{
    return t == bool_type or t == uint8_type or t == uint16_type or t == uint32_type or
           t == uint64_type;
}

double shape::type_max(type_t t)
{
    double r = 0;
    visit_type(t, [&](auto x) { r = static_cast<double>(std::numeric_limits<decltype(x)>::max()); });
    return r;
}

double shape::type_lowest(type_t t)
{
    double r = 0;
    visit_type(t,
               [&](auto x) { r = static_cast<double>(std::numeric_limits<decltype(x)>::lowest()); });
    return r;
}

std::ostream& operator<<(std::ostream& os, const shape& x)
{
    os << x.type_string() << ", {";
    for(std::size_t i = 0; i < x.lens().size(); i++)
        os << (i == 0 ? "" : ", ") << x.lens()[i];
    os << "}, {";
    for(std::size_t i = 0; i < x.strides().size(); i++)
        os << (i == 0 ? "" : ", ") << x.strides()[i];
    os << "}";
    return os;
}

} // namespace migraphx
