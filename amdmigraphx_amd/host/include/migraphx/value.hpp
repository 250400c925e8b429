// A small JSON-like variant used for operator attributes: make_op("slice", {{"axes", {1}}, ...}),
// operation::to_value / from_value.  Follows the construction rules of
// src/include/migraphx/value.hpp: a two-element list whose first element is a string is a
// key/value pair; a list of pairs is an object; any other list is an array.
#ifndef MIGRAPHX_GUARD_VALUE_HPP
#define MIGRAPHX_GUARD_VALUE_HPP

#include <cstdint>
#include <initializer_list>
#include <iosfwd>
#include <string>
#include <type_traits>
#include <vector>
#include <migraphx/errors.hpp>
#include <migraphx/shape.hpp>

namespace migraphx {

struct value
{
    enum kind_t
    {
        null_kind,
        bool_kind,
        int_kind,
        float_kind,
        string_kind,
        array_kind,
        object_kind,
        binary_kind // raw bytes (literal data in a saved program)
    };

    value() = default;
    value(bool b) : m_kind(bool_kind), m_int(b) {}                         // NOLINT
    value(const std::string& s) : m_kind(string_kind), m_str(s) {}         // NOLINT
    value(const char* s) : m_kind(string_kind), m_str(s) {}                // NOLINT
    value(shape::type_t t) : m_kind(int_kind), m_int(t) {}                 // NOLINT
    template <class T,
              std::enable_if_t<std::is_integral<T>{} and not std::is_same<T, bool>{}, int> = 0>
    value(T i) : m_kind(int_kind), m_int(static_cast<int64_t>(i))          // NOLINT
    {
    }
    template <class T, std::enable_if_t<std::is_floating_point<T>{}, int> = 0>
    value(T f) : m_kind(float_kind), m_float(f)                            // NOLINT
    {
    }
    template <class T>
    value(const std::vector<T>& v) : m_kind(array_kind)                    // NOLINT
    {
        for(const auto& x : v)
            m_items.emplace_back(x);
    }
    value(std::initializer_list<value> i);                                 // NOLINT
    value(const std::string& key, const value& v) : value(v) { m_key = key; }

    static value binary(const void* bytes, std::size_t n)
    {
        value v;
        v.m_kind = binary_kind;
        v.m_str.assign(static_cast<const char*>(bytes), n);
        return v;
    }
    static value array() { value v; v.m_kind = array_kind; return v; }
    static value object() { value v; v.m_kind = object_kind; return v; }

    kind_t kind() const { return m_kind; }
    bool is_null() const { return m_kind == null_kind; }
    bool is_string() const { return m_kind == string_kind; }
    bool is_array() const { return m_kind == array_kind; }
    bool is_object() const { return m_kind == object_kind; }
    bool is_binary() const { return m_kind == binary_kind; }
    // the bytes of a binary value
    const std::string& get_binary() const;
    value without_key() const { value v = *this; v.m_key.clear(); return v; }
    bool get_bool() const { return as_int() != 0; }
    int64_t get_int64() const { return as_int(); }
    double get_double() const { return as_float(); }
    const std::string& get_string() const;
    const std::string& get_key() const { return m_key; }

    bool contains(const std::string& key) const;
    const value& at(const std::string& key) const;
    value& operator[](const std::string& key); // inserts into an object
    const value& at(std::size_t i) const;
    std::size_t size() const { return m_items.size(); }
    bool empty() const { return m_items.empty(); }
    const std::vector<value>& items() const { return m_items; }
    void push_back(const value& v);

    template <class T>
    T to() const
    {
        T r{};
        this->get(r);
        return r;
    }
    template <class T>
    std::vector<T> to_vector() const
    {
        return to<std::vector<T>>();
    }

    void get(bool& b) const;
    void get(std::string& s) const;
    void get(shape::type_t& t) const { t = static_cast<shape::type_t>(as_int()); }
    template <class T,
              std::enable_if_t<std::is_integral<T>{} and not std::is_same<T, bool>{}, int> = 0>
    void get(T& i) const
    {
        i = static_cast<T>(as_int());
    }
    template <class T, std::enable_if_t<std::is_floating_point<T>{}, int> = 0>
    void get(T& f) const
    {
        f = static_cast<T>(as_float());
    }
    template <class T>
    void get(std::vector<T>& v) const
    {
        if(m_kind != array_kind and m_kind != object_kind)
            MIGRAPHX_THROW("value: expected an array");
        v.clear();
        for(const auto& x : m_items)
            v.push_back(x.to<T>());
    }

    friend bool operator==(const value& x, const value& y);
    friend bool operator!=(const value& x, const value& y) { return not(x == y); }
    friend std::ostream& operator<<(std::ostream& os, const value& v);

    private:
    int64_t as_int() const;
    double as_float() const;
    kind_t m_kind = null_kind;
    std::string m_key;
    int64_t m_int  = 0;
    double m_float = 0;
    std::string m_str;
    std::vector<value> m_items;
};

} // namespace migraphx
#endif
