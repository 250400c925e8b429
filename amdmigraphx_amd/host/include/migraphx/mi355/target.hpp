// The MI355X target: context (one HIP stream), device memory helpers, the lowering pass and the
// target object registered as "mi355" (interface of src/include/migraphx/target.hpp:130-145;
// the reference's GPU counterpart is src/targets/gpu/target.cpp:243-274).
#ifndef MIGRAPHX_GUARD_MI355_TARGET_HPP
#define MIGRAPHX_GUARD_MI355_TARGET_HPP

#include <memory>
#include <string>
#include <vector>
#include <migraphx/argument.hpp>
#include <migraphx/context.hpp>
#include <migraphx/pass.hpp>
#include <migraphx/target.hpp>

namespace migraphx {
namespace mi355 {

// Owns a HIP stream of default priority; copies share it.  finish() waits for the stream.
struct context
{
    context();
    void* get_stream() const; // hipStream_t
    void finish() const;

    private:
    struct stream_holder;
    std::shared_ptr<stream_holder> m_stream;
};

// device memory of the shape's size, freed with the last copy of the argument
argument allocate_device(const shape& s);
// host -> new device buffer / device -> new host buffer (both wait for the copy)
argument to_device(const argument& host);
argument from_device(const argument& device);

// Replace the operators of the quantized-GEMM path by operators that call the kernel library:
//   quant_dot -> dequantizelinear [-> convert]           one fused mi355::quant_dot
//   dot(x, transpose(dequantizelinear(unpack_int4 ...)))   mi355::w4a16_gemm (MatMulNBits layout)
//   chains of add / sub / mul / div / erf / sqrt / ...     one mi355::chain (fuse_pointwise)
//   quant_dot, dot, quantizelinear, dequantizelinear, unpack_int4, pack_int4, convert, contiguous
//                                                          the mi355:: operator of the same name
// Literals move to device memory, constant subgraphs are evaluated once at compile time, and with
// offload_copy parameters and results are copied in and out.  An operator without a kernel makes
// the pass throw: nothing is ever evaluated on the host.
struct lowering
{
    context* ctx      = nullptr;
    bool offload_copy = false;
    bool fuse_pointwise = true;
    std::string name() const { return "mi355::lowering"; }
    void apply(module& m) const;
};

struct target
{
    std::string name() const { return "mi355"; }
    std::vector<pass> get_passes(migraphx::context& ctx, const compile_options& options) const;
    migraphx::context get_context() const { return context{}; }
    argument copy_to(const argument& a) const { return to_device(a); }
    argument copy_from(const argument& a) const { return from_device(a); }
    argument allocate(const shape& s) const { return allocate_device(s); }
};

} // namespace mi355
} // namespace migraphx
#endif
