// Type-erased operator (src/include/migraphx/operation.hpp:507-555).  A conforming type has
//   std::string name() const;
//   shape compute_shape(std::vector<shape> inputs) const;
// and optionally
//   argument compute(context&, const shape&, const std::vector<argument>&) const;   (target op)
//   argument compute(const shape&, const std::vector<argument>&) const;            (context free)
//   std::ptrdiff_t output_alias(const std::vector<shape>&) const;
//   void finalize(context&, const shape&, const std::vector<shape>&);
//   template <class Self, class F> static void reflect(Self&, F f);   // f(self.member, "member")
//   value to_value() const; void from_value(const value&);            // instead of reflect
//   value attributes() const;
// reflect gives to_value / from_value, equality and printing.
#ifndef MIGRAPHX_GUARD_OPERATION_HPP
#define MIGRAPHX_GUARD_OPERATION_HPP

#include <memory>
#include <ostream>
#include <sstream>
#include <string>
#include <typeinfo>
#include <vector>
#include <migraphx/argument.hpp>
#include <migraphx/context.hpp>
#include <migraphx/serialize.hpp>
#include <migraphx/value.hpp>

namespace migraphx {

namespace detail {

template <class...>
using void_t = void;

template <class T, class = void>
struct has_reflect : std::false_type {};
struct reflect_probe
{
    template <class U>
    void operator()(U&, const char*) const
    {
    }
};
template <class T>
struct has_reflect<T, void_t<decltype(T::reflect(std::declval<T&>(), reflect_probe{}))>>
    : std::true_type {};

template <class T, class = void>
struct has_ctx_compute : std::false_type {};
template <class T>
struct has_ctx_compute<T,
                       void_t<decltype(std::declval<const T&>().compute(
                           std::declval<context&>(),
                           std::declval<const shape&>(),
                           std::declval<const std::vector<argument>&>()))>> : std::true_type {};

template <class T, class = void>
struct has_free_compute : std::false_type {};
template <class T>
struct has_free_compute<T,
                        void_t<decltype(std::declval<const T&>().compute(
                            std::declval<const shape&>(),
                            std::declval<const std::vector<argument>&>()))>> : std::true_type {};

template <class T, class = void>
struct has_output_alias : std::false_type {};
template <class T>
struct has_output_alias<T,
                        void_t<decltype(std::declval<const T&>().output_alias(
                            std::declval<const std::vector<shape>&>()))>> : std::true_type {};

template <class T, class = void>
struct has_finalize : std::false_type {};
template <class T>
struct has_finalize<T,
                    void_t<decltype(std::declval<T&>().finalize(
                        std::declval<context&>(),
                        std::declval<const shape&>(),
                        std::declval<const std::vector<shape>&>()))>> : std::true_type {};

template <class T, class = void>
struct has_attributes : std::false_type {};
template <class T>
struct has_attributes<T, void_t<decltype(std::declval<const T&>().attributes())>> : std::true_type {};

// a type may write and read its fields itself: value to_value() const; void from_value(const value&)
template <class T, class = void>
struct has_own_value : std::false_type {};
template <class T>
struct has_own_value<T,
                     void_t<decltype(std::declval<const T&>().to_value()),
                            decltype(std::declval<T&>().from_value(std::declval<const value&>()))>>
    : std::true_type {};

struct to_value_visitor
{
    value* v;
    template <class U>
    void operator()(const U& x, const char* name) const
    {
        (*v)[name] = value(std::string(name), migraphx::to_value(x));
    }
};

struct from_value_visitor
{
    const value* v;
    template <class U>
    void operator()(U& x, const char* name) const
    {
        if(v->contains(name))
            migraphx::from_value(v->at(name), x);
    }
};

} // namespace detail

struct operation
{
    operation() = default;
    template <class T, std::enable_if_t<not std::is_same<std::decay_t<T>, operation>{}, int> = 0>
    operation(T x) : m_impl(std::make_shared<model<T>>(std::move(x))) // NOLINT
    {
    }
    operation(const operation& o) : m_impl(o.m_impl ? o.m_impl->clone() : nullptr) {}
    operation(operation&&) noexcept = default;
    operation& operator=(operation o)
    {
        std::swap(m_impl, o.m_impl);
        return *this;
    }

    std::string name() const { return get().name(); }
    shape compute_shape(const std::vector<shape>& inputs) const { return get().compute_shape(inputs); }
    bool is_context_free() const { return get().is_context_free(); }
    bool has_compute() const { return get().has_compute(); }
    argument compute(context& ctx, const shape& out, const std::vector<argument>& args) const
    {
        return get().compute(ctx, out, args);
    }
    argument compute(const shape& out, const std::vector<argument>& args) const
    {
        return get().compute(out, args);
    }
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return get().output_alias(s); }
    void finalize(context& ctx, const shape& out, const std::vector<shape>& in)
    {
        if(m_impl)
            m_impl->finalize(ctx, out, in);
    }
    value to_value() const { return get().to_value(); }
    void from_value(const value& v) { m_impl->from_value(v); }
    value attributes() const { return get().attributes(); }
    bool empty() const { return m_impl == nullptr; }

    template <class T>
    T* any_cast()
    {
        if(not m_impl or m_impl->type() != typeid(T))
            return nullptr;
        return static_cast<T*>(m_impl->ptr());
    }
    template <class T>
    const T* any_cast() const
    {
        return const_cast<operation*>(this)->any_cast<T>();
    }

    friend bool operator==(const operation& x, const operation& y)
    {
        return x.name() == y.name() and x.to_value() == y.to_value();
    }
    friend bool operator!=(const operation& x, const operation& y) { return not(x == y); }
    friend std::ostream& operator<<(std::ostream& os, const operation& op)
    {
        os << op.name();
        auto v = op.to_value();
        if(not v.empty())
        {
            os << "[";
            for(std::size_t i = 0; i < v.size(); i++)
                os << (i == 0 ? "" : ",") << v.items()[i].get_key() << "=" << v.items()[i];
            os << "]";
        }
        return os;
    }

    private:
    struct base
    {
        virtual ~base()                                                              = default;
        virtual std::shared_ptr<base> clone() const                                  = 0;
        virtual std::string name() const                                             = 0;
        virtual shape compute_shape(const std::vector<shape>&) const                 = 0;
        virtual bool is_context_free() const                                         = 0;
        virtual bool has_compute() const                                             = 0;
        virtual argument compute(context&, const shape&, const std::vector<argument>&) const = 0;
        virtual argument compute(const shape&, const std::vector<argument>&) const   = 0;
        virtual std::ptrdiff_t output_alias(const std::vector<shape>&) const         = 0;
        virtual void finalize(context&, const shape&, const std::vector<shape>&)     = 0;
        virtual value to_value() const                                               = 0;
        virtual void from_value(const value&)                                        = 0;
        virtual value attributes() const                                             = 0;
        virtual void* ptr()                                                          = 0;
        virtual const std::type_info& type() const                                   = 0;
    };

    template <class T>
    struct model : base
    {
        T x;
        explicit model(T v) : x(std::move(v)) {}
        std::shared_ptr<base> clone() const override { return std::make_shared<model<T>>(x); }
        std::string name() const override { return x.name(); }
        shape compute_shape(const std::vector<shape>& in) const override { return x.compute_shape(in); }
        bool is_context_free() const override { return detail::has_free_compute<T>{}; }
        bool has_compute() const override
        {
            return detail::has_free_compute<T>{} or detail::has_ctx_compute<T>{};
        }
        argument
        compute(context& ctx, const shape& out, const std::vector<argument>& args) const override
        {
            if constexpr(detail::has_ctx_compute<T>{})
                return x.compute(ctx, out, args);
            else if constexpr(detail::has_free_compute<T>{})
                return x.compute(out, args);
            else
                MIGRAPHX_THROW("Not computable: " + x.name());
        }
        argument compute(const shape& out, const std::vector<argument>& args) const override
        {
            if constexpr(detail::has_free_compute<T>{})
                return x.compute(out, args);
            else
                MIGRAPHX_THROW("Not computable without a context: " + x.name());
        }
        std::ptrdiff_t output_alias(const std::vector<shape>& s) const override
        {
            if constexpr(detail::has_output_alias<T>{})
                return x.output_alias(s);
            else
                return -1;
        }
        void finalize(context& ctx, const shape& out, const std::vector<shape>& in) override
        {
            if constexpr(detail::has_finalize<T>{})
                x.finalize(ctx, out, in);
        }
        value to_value() const override
        {
            value v = value::object();
            if constexpr(detail::has_own_value<T>{})
                v = x.to_value();
            else if constexpr(detail::has_reflect<T>{})
                T::reflect(x, detail::to_value_visitor{&v});
            return v;
        }
        void from_value(const value& v) override
        {
            if constexpr(detail::has_own_value<T>{})
                x.from_value(v);
            else if constexpr(detail::has_reflect<T>{})
                T::reflect(x, detail::from_value_visitor{&v});
        }
        value attributes() const override
        {
            if constexpr(detail::has_attributes<T>{})
                return x.attributes();
            else
                return value::object();
        }
        void* ptr() override { return &x; }
        const std::type_info& type() const override { return typeid(T); }
    };

    const base& get() const
    {
        if(not m_impl)
            MIGRAPHX_THROW("empty operation");
        return *m_impl;
    }
    std::shared_ptr<base> m_impl;
};

template <class T>
T& any_cast(operation& op)
{
    auto* p = op.any_cast<T>();
    if(p == nullptr)
        MIGRAPHX_THROW("operation: bad any_cast from " + op.name());
    return *p;
}
template <class T>
const T& any_cast(const operation& op)
{
    const auto* p = op.any_cast<T>();
    if(p == nullptr)
        MIGRAPHX_THROW("operation: bad any_cast from " + op.name());
    return *p;
}

} // namespace migraphx
#endif
