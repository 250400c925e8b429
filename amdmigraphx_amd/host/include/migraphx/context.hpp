// Type-erased execution context: any copyable type with `void finish() const`
// (src/include/migraphx/context.hpp:45-49).
#ifndef MIGRAPHX_GUARD_CONTEXT_HPP
#define MIGRAPHX_GUARD_CONTEXT_HPP

#include <memory>
#include <typeinfo>
#include <migraphx/errors.hpp>

namespace migraphx {

struct context
{
    context() = default;
    template <class T, std::enable_if_t<not std::is_same<std::decay_t<T>, context>{}, int> = 0>
    context(T x) : m_impl(std::make_shared<model<T>>(std::move(x))) // NOLINT
    {
    }
    void finish() const
    {
        if(m_impl)
            m_impl->finish();
    }
    bool empty() const { return m_impl == nullptr; }
    template <class T>
    T* any_cast()
    {
        if(not m_impl or m_impl->type() != typeid(T))
            return nullptr;
        return static_cast<T*>(m_impl->ptr());
    }

    private:
    struct base
    {
        virtual ~base()                             = default;
        virtual void finish() const                 = 0;
        virtual void* ptr()                         = 0;
        virtual const std::type_info& type() const  = 0;
    };
    template <class T>
    struct model : base
    {
        T x;
        explicit model(T v) : x(std::move(v)) {}
        void finish() const override { x.finish(); }
        void* ptr() override { return &x; }
        const std::type_info& type() const override { return typeid(T); }
    };
    std::shared_ptr<base> m_impl; // shared: a program and its copies drive one stream
};

template <class T>
T& any_cast(context& c)
{
    auto* p = c.any_cast<T>();
    if(p == nullptr)
        MIGRAPHX_THROW("context: wrong context type for this target");
    return *p;
}

} // namespace migraphx
#endif
