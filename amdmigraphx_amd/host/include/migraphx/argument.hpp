// argument: a shape plus shared ownership of the bytes it describes (host or device memory).
// literal: an argument that owns host bytes and compares by value.
// Follows src/include/migraphx/argument.hpp:51-121 and literal.hpp: copies share the buffer, a view
// operator returns the same buffer under another shape, operators never free their inputs.
#ifndef MIGRAPHX_GUARD_ARGUMENT_HPP
#define MIGRAPHX_GUARD_ARGUMENT_HPP

#include <cstring>
#include <iosfwd>
#include <memory>
#include <vector>
#include <migraphx/shape.hpp>

namespace migraphx {

// typed, strided view over an argument's memory; iteration is in logical (row-major) order
template <class T>
struct tensor_view
{
    T* base = nullptr;
    shape s;
    std::size_t size() const { return s.elements(); }
    T& operator[](std::size_t i) const { return base[s.index(i)]; }
    const shape& get_shape() const { return s; }
    struct iterator
    {
        const tensor_view* v;
        std::size_t i;
        T& operator*() const { return (*v)[i]; }
        iterator& operator++() { ++i; return *this; }
        bool operator!=(const iterator& o) const { return i != o.i; }
        bool operator==(const iterator& o) const { return i == o.i; }
    };
    iterator begin() const { return {this, 0}; }
    iterator end() const { return {this, size()}; }
};

struct argument
{
    argument() = default;
    // allocate zeroed host memory for s
    explicit argument(const shape& s);
    // non-owning view of existing memory
    argument(const shape& s, void* p) : m_shape(s), m_data(std::shared_ptr<char>(), static_cast<char*>(p)) {}
    // shared ownership
    argument(const shape& s, std::shared_ptr<char> p) : m_shape(s), m_data(std::move(p)) {}

    template <class T>
    argument(const shape& s, const std::vector<T>& v) : argument(s)
    {
        fill(v);
    }

    char* data() const { return m_data.get(); }
    const shape& get_shape() const { return m_shape; }
    bool empty() const { return m_data == nullptr; }
    // same memory under another shape
    argument reshape(const shape& s) const { return {s, m_data}; }
    // same memory, starting `bytes` further
    argument offset(std::size_t bytes, const shape& s) const
    {
        return {s, std::shared_ptr<char>(m_data, m_data.get() + bytes)};
    }
    const std::shared_ptr<char>& share() const { return m_data; }

    template <class T>
    tensor_view<T> get() const
    {
        if(shape::get_type<T>::value != m_shape.type())
            MIGRAPHX_THROW("argument::get: element type mismatch");
        return {reinterpret_cast<T*>(m_data.get()), m_shape};
    }

    // f(tensor_view<T>) with the argument's element type
    template <class F>
    void visit(F f) const
    {
        visit_type(m_shape.type(), [&](auto x) { f(this->get<decltype(x)>()); });
    }

    // elements in logical order, converted to T
    template <class T>
    std::vector<T> to_vector() const
    {
        std::vector<T> r;
        r.reserve(m_shape.elements());
        visit([&](auto v) {
            for(std::size_t i = 0; i < v.size(); i++)
                r.push_back(static_cast<T>(static_cast<double>(v[i])));
        });
        return r;
    }

    // fill in logical order from values of any arithmetic type
    template <class T>
    void fill(const std::vector<T>& v)
    {
        if(v.size() != m_shape.elements())
            MIGRAPHX_THROW("argument: " + std::to_string(v.size()) + " values for " +
                           std::to_string(m_shape.elements()) + " elements");
        visit([&](auto out) {
            using O = std::remove_reference_t<decltype(out[0])>;
            for(std::size_t i = 0; i < v.size(); i++)
                out[i] = O(v[i]);
        });
    }

    friend std::ostream& operator<<(std::ostream& os, const argument& a);

    private:
    shape m_shape;
    std::shared_ptr<char> m_data;
};

struct literal
{
    literal() = default;
    template <class T>
    literal(const shape& s, const std::vector<T>& v) : m_arg(s, v)
    {
    }
    template <class T>
    literal(const shape& s, std::initializer_list<T> v) : literal(s, std::vector<T>(v))
    {
    }
    // raw bytes in memory order
    literal(const shape& s, const char* bytes) : m_arg(s)
    {
        std::memcpy(m_arg.data(), bytes, s.bytes());
    }
    // scalar
    template <class T, std::enable_if_t<std::is_arithmetic<T>{}, int> = 0>
    literal(T x) : literal(shape{shape::get_type<T>::value}, std::vector<T>{x}) // NOLINT
    {
    }

    const shape& get_shape() const { return m_arg.get_shape(); }
    const char* data() const { return m_arg.data(); }
    bool empty() const { return m_arg.empty(); }
    argument get_argument() const { return m_arg; }
    template <class F>
    void visit(F f) const
    {
        m_arg.visit(f);
    }
    template <class T>
    T at(std::size_t i = 0) const
    {
        return m_arg.to_vector<T>().at(i);
    }
    friend bool operator==(const literal& x, const literal& y);
    friend bool operator!=(const literal& x, const literal& y) { return not(x == y); }
    friend std::ostream& operator<<(std::ostream& os, const literal& l) { return os << l.m_arg; }

    private:
    argument m_arg;
};

} // namespace migraphx
#endif
