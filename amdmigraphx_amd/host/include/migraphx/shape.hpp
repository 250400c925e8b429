// Tensor shape: element type, dimensions and element strides.
// Mirrors the static-shape part of src/include/migraphx/shape.hpp (type list :57-73, predicates
// standard / packed / transposed / broadcasted / scalar, index and multi-index arithmetic).
#ifndef MIGRAPHX_GUARD_SHAPE_HPP
#define MIGRAPHX_GUARD_SHAPE_HPP

#include <cstddef>
#include <cstdint>
#include <initializer_list>
#include <iosfwd>
#include <string>
#include <vector>
#include <migraphx/errors.hpp>
#include <migraphx/float_types.hpp>

namespace migraphx {

// clang-format off
#define MIGRAPHX_SHAPE_VISIT_TYPES(m) \
    m(bool_type, bool) \
    m(half_type, migraphx::half) \
    m(float_type, float) \
    m(double_type, double) \
    m(uint8_type, uint8_t) \
    m(int8_type, int8_t) \
    m(uint16_type, uint16_t) \
    m(int16_type, int16_t) \
    m(int32_type, int32_t) \
    m(int64_type, int64_t) \
    m(uint32_type, uint32_t) \
    m(uint64_type, uint64_t) \
    m(fp8e4m3fn_type, migraphx::fp8e4m3fn) \
    m(fp8e5m2_type, migraphx::fp8e5m2) \
    m(bf16_type, migraphx::bf16)
// clang-format on

struct shape
{
    // numbering of the reference's enum (shape.hpp:57-73); the fnuz fp8 variants keep their
    // slots but no kernel of this build takes them
    enum type_t
    {
        bool_type        = 0,
        half_type        = 1,
        float_type       = 2,
        double_type      = 3,
        uint8_type       = 4,
        int8_type        = 5,
        uint16_type      = 6,
        int16_type       = 7,
        int32_type       = 8,
        int64_type       = 9,
        uint32_type      = 10,
        uint64_type      = 11,
        fp8e4m3fnuz_type = 12,
        fp8e4m3fn_type   = 13,
        fp8e5m2_type     = 14,
        bf16_type        = 15,
        fp8e5m2fnuz_type = 16,
        tuple_type       = 17,
        fp4x2_type       = 18 // two e2m1 values packed in a byte, low nibble first; not visitable
    };

    template <class T>
    struct get_type;

    shape() = default;
    shape(type_t t) : m_type(t), m_lens({1}), m_strides({0}) {} // NOLINT
    shape(type_t t, std::vector<std::size_t> l);
    shape(type_t t, std::vector<std::size_t> l, std::vector<std::size_t> s);
    shape(type_t t, std::initializer_list<std::size_t> l) : shape(t, std::vector<std::size_t>(l)) {}

    // lens permuted so that the memory order follows `perm` (shape.hpp from_permutation)
    static shape
    from_permutation(type_t t, const std::vector<std::size_t>& l, const std::vector<int64_t>& perm);

    type_t type() const { return m_type; }
    const std::vector<std::size_t>& lens() const { return m_lens; }
    const std::vector<std::size_t>& strides() const { return m_strides; }
    std::size_t ndim() const { return m_lens.size(); }
    std::size_t elements() const;
    std::size_t bytes() const { return element_space() * type_size(); }
    std::size_t type_size() const { return type_size(m_type); }
    static std::size_t type_size(type_t t);
    // number of elements the addressed memory spans
    std::size_t element_space() const;

    std::size_t index(const std::vector<std::size_t>& multi) const;
    // memory offset of the i-th element in logical (row-major) order
    std::size_t index(std::size_t i) const;
    std::vector<std::size_t> multi(std::size_t i) const;

    bool packed() const;      // no holes in memory
    bool transposed() const;  // packed but strides not descending
    bool broadcasted() const; // some stride is zero
    bool standard() const;    // packed, row-major
    bool scalar() const;      // all strides zero
    bool empty() const { return m_lens.empty(); }

    shape normalize_standard() const;
    shape with_lens(type_t t, const std::vector<std::size_t>& l) const;
    shape with_lens(const std::vector<std::size_t>& l) const { return with_lens(m_type, l); }
    shape with_type(type_t t) const;
    shape as_standard() const { return {m_type, m_lens}; }

    std::string type_string() const { return type_name(m_type); }
    static std::string type_name(type_t t);
    static type_t parse_type(const std::string& s);
    static bool is_integral(type_t t);
    static bool is_unsigned(type_t t);
    // largest / smallest finite value of the type, as the reference's shape::as<T>::max()/min()
    static double type_max(type_t t);
    static double type_lowest(type_t t);

    friend bool operator==(const shape& x, const shape& y)
    {
        return x.m_type == y.m_type and x.m_lens == y.m_lens and x.m_strides == y.m_strides;
    }
    friend bool operator!=(const shape& x, const shape& y) { return not(x == y); }
    friend std::ostream& operator<<(std::ostream& os, const shape& x);

    private:
    type_t m_type = float_type;
    std::vector<std::size_t> m_lens;
    std::vector<std::size_t> m_strides;
    void calculate_strides();
};

#define MIGRAPHX_SHAPE_GET_TYPE(x, t)                         \
    template <>                                               \
    struct shape::get_type<t>                                 \
    {                                                         \
        static constexpr shape::type_t value = shape::x;      \
    };
MIGRAPHX_SHAPE_VISIT_TYPES(MIGRAPHX_SHAPE_GET_TYPE)
#undef MIGRAPHX_SHAPE_GET_TYPE

// call f(T{}) with the C++ type of t
template <class F>
void visit_type(shape::type_t t, F f)
{
    switch(t)
    {
#define MIGRAPHX_SHAPE_VISIT_CASE(x, T) \
    case shape::x: f(T{}); return;
        MIGRAPHX_SHAPE_VISIT_TYPES(MIGRAPHX_SHAPE_VISIT_CASE)
#undef MIGRAPHX_SHAPE_VISIT_CASE
    default: MIGRAPHX_THROW("visit_type: type " + shape::type_name(t) + " has no host representation");
    }
}

} // namespace migraphx
#endif
