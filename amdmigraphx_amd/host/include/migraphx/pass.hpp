// Type-erased pass (src/include/migraphx/pass.hpp): `std::string name() const` and
// `void apply(module&) const`.  run_passes validates the module after every pass.
#ifndef MIGRAPHX_GUARD_PASS_HPP
#define MIGRAPHX_GUARD_PASS_HPP

#include <memory>
#include <string>
#include <vector>
#include <migraphx/module.hpp>

namespace migraphx {

struct program;

struct pass
{
    template <class T, std::enable_if_t<not std::is_same<std::decay_t<T>, pass>{}, int> = 0>
    pass(T x) : m_impl(std::make_shared<model<T>>(std::move(x))) // NOLINT
    {
    }
    std::string name() const { return m_impl->name(); }
    void apply(module& m) const { m_impl->apply(m); }

    private:
    struct base
    {
        virtual ~base()                       = default;
        virtual std::string name() const      = 0;
        virtual void apply(module& m) const   = 0;
    };
    template <class T>
    struct model : base
    {
        T x;
        explicit model(T v) : x(std::move(v)) {}
        std::string name() const override { return x.name(); }
        void apply(module& m) const override { x.apply(m); }
    };
    std::shared_ptr<base> m_impl;
};

void run_passes(module& m, const std::vector<pass>& passes);
void run_passes(program& p, const std::vector<pass>& passes);

} // namespace migraphx
#endif
