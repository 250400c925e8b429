#include <migraphx/argument.hpp>
#include <ostream>

namespace migraphx {

argument::argument(const shape& s) : m_shape(s)
{
    const std::size_t n = s.bytes();
    // one spare byte so that an empty tensor still owns a distinct address
    m_data = std::shared_ptr<char>(new char[n + 1](), std::default_delete<char[]>());
}

std::ostream& operator<<(std::ostream& os, const argument& a)
{
    if(a.empty())
        return os << "{}";
    if(a.get_shape().type() == shape::fp4x2_type)
    {
        // packed fp4 has no element type to visit: show the bytes
        const std::size_t nb = a.get_shape().bytes();
        for(std::size_t i = 0; i < nb and i < 16; i++)
            os << (i == 0 ? "0x" : ", 0x") << std::hex << (static_cast<unsigned>(a.data()[i]) & 0xffu) << std::dec;
        if(nb > 16)
            os << ", ...";
        return os;
    }
    const auto v        = a.to_vector<double>();
    const std::size_t n = v.size() > 16 ? 16 : v.size();
    for(std::size_t i = 0; i < n; i++)
        os << (i == 0 ? "" : ", ") << v[i];
    if(n < v.size())
        os << ", ...";
    return os;
}

bool operator==(const literal& x, const literal& y)
{
    if(x.get_shape() != y.get_shape())
        return false;
    if(x.empty() or y.empty())
        return x.empty() == y.empty();
    return std::memcmp(x.data(), y.data(), x.get_shape().bytes()) == 0;
}

} // namespace migraphx
