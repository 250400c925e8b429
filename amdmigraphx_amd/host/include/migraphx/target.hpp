// Type-erased target (src/include/migraphx/target.hpp:130-145): name, the passes that lower a
// program for it, its context, and how tensors reach and leave its memory.  A target type may
// leave out copy_to / copy_from / allocate; the defaults keep tensors in host memory (:102-126).
#ifndef MIGRAPHX_GUARD_TARGET_HPP
#define MIGRAPHX_GUARD_TARGET_HPP

#include <memory>
#include <string>
#include <vector>
#include <migraphx/argument.hpp>
#include <migraphx/context.hpp>
#include <migraphx/pass.hpp>

namespace migraphx {

struct compile_options
{
    // copy parameters to the target's memory and results back inside eval
    bool offload_copy = false;
    bool fast_math    = true;
    bool exhaustive_tune = false;
};

namespace detail {
template <class T, class = void>
struct has_copy_to : std::false_type {};
template <class T>
struct has_copy_to<T, void_t<decltype(std::declval<const T&>().copy_to(std::declval<const argument&>()))>>
    : std::true_type {};
template <class T, class = void>
struct has_copy_from : std::false_type {};
template <class T>
struct has_copy_from<T, void_t<decltype(std::declval<const T&>().copy_from(std::declval<const argument&>()))>>
    : std::true_type {};
template <class T, class = void>
struct has_allocate : std::false_type {};
template <class T>
struct has_allocate<T, void_t<decltype(std::declval<const T&>().allocate(std::declval<const shape&>()))>>
    : std::true_type {};
} // namespace detail

struct target
{
    target() = default;
    template <class T, std::enable_if_t<not std::is_same<std::decay_t<T>, target>{}, int> = 0>
    target(T x) : m_impl(std::make_shared<model<T>>(std::move(x))) // NOLINT
    {
    }
    std::string name() const { return get().name(); }
    std::vector<pass> get_passes(context& ctx, const compile_options& o) const
    {
        return get().get_passes(ctx, o);
    }
    context get_context() const { return get().get_context(); }
    argument copy_to(const argument& a) const { return get().copy_to(a); }
    argument copy_from(const argument& a) const { return get().copy_from(a); }
    argument allocate(const shape& s) const { return get().allocate(s); }
    bool empty() const { return m_impl == nullptr; }

    private:
    struct base
    {
        virtual ~base()                                                              = default;
        virtual std::string name() const                                             = 0;
        virtual std::vector<pass> get_passes(context&, const compile_options&) const = 0;
        virtual context get_context() const                                          = 0;
        virtual argument copy_to(const argument&) const                              = 0;
        virtual argument copy_from(const argument&) const                            = 0;
        virtual argument allocate(const shape&) const                                = 0;
    };
    template <class T>
    struct model : base
    {
        T x;
        explicit model(T v) : x(std::move(v)) {}
        std::string name() const override { return x.name(); }
        std::vector<pass> get_passes(context& c, const compile_options& o) const override
        {
            return x.get_passes(c, o);
        }
        context get_context() const override { return x.get_context(); }
        argument copy_to(const argument& a) const override
        {
            if constexpr(detail::has_copy_to<T>{})
                return x.copy_to(a);
            else
                return a;
        }
        argument copy_from(const argument& a) const override
        {
            if constexpr(detail::has_copy_from<T>{})
                return x.copy_from(a);
            else
                return a;
        }
        argument allocate(const shape& s) const override
        {
            if constexpr(detail::has_allocate<T>{})
                return x.allocate(s);
            else
                return argument{s};
        }
    };
    const base& get() const
    {
        if(not m_impl)
            MIGRAPHX_THROW("empty target");
        return *m_impl;
    }
    std::shared_ptr<base> m_impl;
};

} // namespace migraphx
#endif
