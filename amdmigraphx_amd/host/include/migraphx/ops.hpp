// The operators on the quantized-GEMM path and the view operators around them.
// Shape rules follow the reference operator of the same name (file:line at each struct).
// Arithmetic operators carry no host `compute`: a target lowers them to its own kernels, and a
// program that still holds one after lowering cannot be evaluated.  View operators (transpose,
// broadcasts, squeeze / unsqueeze, slice, reshape of a standard tensor) are context free: they
// return the input's memory under the new shape, on the host or on a device alike.
#ifndef MIGRAPHX_GUARD_OPS_HPP
#define MIGRAPHX_GUARD_OPS_HPP

#include <functional>
#include <string>
#include <vector>
#include <migraphx/operation.hpp>

namespace migraphx {
namespace op {

// src/include/migraphx/op/quant_dot.hpp:51-121
struct quant_dot
{
    value attributes() const { return {{"general_data_type", "dot"}}; }
    std::string name() const { return "quant_dot"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/dot.hpp:44-100
struct dot
{
    std::string name() const { return "dot"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// Attributes and shape rule shared by convolution and quant_convolution
// (src/include/migraphx/op/quant_convolution.hpp:52-134, op/convolution.hpp:47-206): input
// [N, C, spatial...], weights [O, C / group, window...]; `padding` holds one entry per spatial
// dimension (both sides) or two (all the left ones, then all the right ones).
struct convolution_attributes
{
    std::vector<int64_t> padding  = {0, 0};
    std::vector<int64_t> stride   = {1, 1};
    std::vector<int64_t> dilation = {1, 1};
    int64_t padding_mode          = 0; // default_: the padding that is given
    int64_t group                 = 1;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.padding, "padding");
        f(self.stride, "stride");
        f(self.dilation, "dilation");
        f(self.padding_mode, "padding_mode");
        f(self.group, "group");
    }
    std::size_t kdims() const;
    std::vector<std::size_t> output_lens(const std::string& opname, const shape& input, const shape& weights) const;
};

// src/include/migraphx/op/convolution.hpp:47-206 (static shapes)
struct convolution : convolution_attributes
{
    std::string name() const { return "convolution"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/quant_convolution.hpp:52-134: int8 -> int32, fp8 / float / fp4x2 -> float
struct quant_convolution : convolution_attributes
{
    value attributes() const { return {{"general_data_type", "convolution"}}; }
    std::string name() const { return "quant_convolution"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/quantizelinear.hpp:50-69
struct quantizelinear
{
    int64_t out_type = -1; // shape::type_t, or -1: the zero point's type, uint8 without one
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.out_type, "out_type");
    }
    value attributes() const { return {{"pointwise", true}}; }
    std::string name() const { return "quantizelinear"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/dequantizelinear.hpp:40-58
struct dequantizelinear
{
    value attributes() const { return {{"pointwise", true}}; }
    std::string name() const { return "dequantizelinear"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/unpack_int4.hpp:43-73
struct unpack_int4
{
    int64_t axis = -1;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axis, "axis");
    }
    std::string name() const { return "unpack_int4"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/pack_int4.hpp:44-77
struct pack_int4
{
    int64_t axis = -1;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axis, "axis");
    }
    std::string name() const { return "pack_int4"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/unpack_fp4.hpp:42-76: fp4x2 -> fp8e4m3fn, the axis doubled
struct unpack_fp4
{
    int64_t axis = -1;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axis, "axis");
    }
    std::string name() const { return "unpack_fp4"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/pack_fp4.hpp:43-80: any arithmetic type -> fp4x2, the axis halved
struct pack_fp4
{
    int64_t axis = -1;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axis, "axis");
    }
    std::string name() const { return "pack_fp4"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/convert.hpp:40-62
struct convert
{
    shape::type_t target_type = shape::half_type;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.target_type, "target_type");
    }
    value attributes() const { return {{"pointwise", true}}; }
    std::string name() const { return "convert"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/binary.hpp:60-90 (mul.hpp, add.hpp, sub.hpp)
struct binary
{
    std::string op_name;
    std::string name() const { return op_name; }
    value attributes() const { return {{"pointwise", true}}; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};
struct mul : binary { mul() : binary{"mul"} {} };
struct add : binary { add() : binary{"add"} {} };
struct sub : binary { sub() : binary{"sub"} {} };
struct div : binary { div() : binary{"div"} {} };
struct max : binary { max() : binary{"max"} {} }; // op/max.hpp: std::max(x, y)
struct min : binary { min() : binary{"min"} {} }; // op/min.hpp: std::min(x, y)

// src/include/migraphx/op/unary.hpp (erf.hpp, sqrt.hpp, rsqrt.hpp, exp.hpp, tanh.hpp, neg.hpp): the
// result has the input's shape
struct unary
{
    std::string op_name;
    std::string name() const { return op_name; }
    value attributes() const { return {{"pointwise", true}}; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};
struct erf : unary { erf() : unary{"erf"} {} };
struct sqrt : unary { sqrt() : unary{"sqrt"} {} };
struct rsqrt : unary { rsqrt() : unary{"rsqrt"} {} };
struct exp : unary { exp() : unary{"exp"} {} };
struct tanh : unary { tanh() : unary{"tanh"} {} };
struct neg : unary { neg() : unary{"neg"} {} };
struct nearbyint : unary { nearbyint() : unary{"nearbyint"} {} }; // op/nearbyint.hpp: ties to even

// src/include/migraphx/op/reduce_mean.hpp:34-50, reduce_op.hpp:80-180: reduced axes keep length 1
struct reduce_mean
{
    std::vector<int64_t> axes;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axes, "axes");
    }
    std::string name() const { return "reduce_mean"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/reduce_max.hpp, reduce_min.hpp (reduce_op.hpp:80-180): as reduce_mean
struct reduce_extreme
{
    std::string op_name;
    std::vector<int64_t> axes;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axes, "axes");
    }
    std::string name() const { return op_name; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};
struct reduce_max : reduce_extreme { reduce_max() : reduce_extreme{"reduce_max", {}} {} };
struct reduce_min : reduce_extreme { reduce_min() : reduce_extreme{"reduce_min", {}} {} };

// src/include/migraphx/op/clip.hpp:44-70: min(max(lowest, x), highest), the three inputs of one shape
struct clip
{
    std::string name() const { return "clip"; }
    value attributes() const { return {{"pointwise", true}}; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/softmax.hpp:36-60
struct softmax
{
    int64_t axis = 1;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axis, "axis");
    }
    std::string name() const { return "softmax"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/gather.hpp:42-98
struct gather
{
    int64_t axis = 0;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axis, "axis");
    }
    std::string name() const { return "gather"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
};

// src/include/migraphx/op/broadcast.hpp:52-128
struct broadcast
{
    uint64_t axis = 0;
    std::vector<std::size_t> out_lens;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axis, "axis");
        f(self.out_lens, "out_lens");
    }
    std::string name() const { return "broadcast"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(const shape& out, const std::vector<argument>& args) const
    {
        return args.at(0).reshape(out);
    }
    std::ptrdiff_t output_alias(const std::vector<shape>&) const { return 0; }
};

// src/include/migraphx/op/multibroadcast.hpp:45-127
struct multibroadcast
{
    std::vector<std::size_t> out_lens;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.out_lens, "out_lens");
    }
    std::string name() const { return "multibroadcast"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(const shape& out, const std::vector<argument>& args) const
    {
        return args.at(0).reshape(out);
    }
    std::ptrdiff_t output_alias(const std::vector<shape>&) const { return 0; }
};

// src/include/migraphx/op/transpose.hpp:43-111
struct transpose
{
    std::vector<int64_t> permutation;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.permutation, "permutation");
    }
    std::string name() const { return "transpose"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(const shape& out, const std::vector<argument>& args) const
    {
        return args.at(0).reshape(out);
    }
    std::ptrdiff_t output_alias(const std::vector<shape>&) const { return 0; }
};

// src/include/migraphx/op/reshape.hpp:44-260.  The result is a standard tensor; the host
// `compute` exists for standard inputs only (same bytes, new dimensions).
struct reshape
{
    std::vector<int64_t> dims;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.dims, "dims");
    }
    std::string name() const { return "reshape"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(const shape& out, const std::vector<argument>& args) const;
};

// src/include/migraphx/op/unsqueeze.hpp:44-140
struct unsqueeze
{
    std::vector<int64_t> axes;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axes, "axes");
    }
    std::string name() const { return "unsqueeze"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(const shape& out, const std::vector<argument>& args) const
    {
        return args.at(0).reshape(out);
    }
    std::ptrdiff_t output_alias(const std::vector<shape>&) const { return 0; }
};

// src/include/migraphx/op/squeeze.hpp:43-130
struct squeeze
{
    std::vector<int64_t> axes;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axes, "axes");
    }
    std::string name() const { return "squeeze"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(const shape& out, const std::vector<argument>& args) const
    {
        return args.at(0).reshape(out);
    }
    std::ptrdiff_t output_alias(const std::vector<shape>&) const { return 0; }
};

// src/include/migraphx/op/slice.hpp:47-300 (constant axes / starts / ends)
struct slice
{
    std::vector<int64_t> axes;
    std::vector<int64_t> starts;
    std::vector<int64_t> ends;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axes, "axes");
        f(self.starts, "starts");
        f(self.ends, "ends");
    }
    std::string name() const { return "slice"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    std::size_t compute_offset(const shape& in) const; // in elements
    argument compute(const shape& out, const std::vector<argument>& args) const
    {
        const auto& in = args.at(0).get_shape();
        return args[0].offset(compute_offset(in) * in.type_size(), out);
    }
    std::ptrdiff_t output_alias(const std::vector<shape>&) const { return 0; }
};

// src/include/migraphx/op/contiguous.hpp:43-83: standard-layout copy.  The host compute serves
// compile-time evaluation of literals; targets lower it to their own copy kernel.
struct contiguous
{
    std::string name() const { return "contiguous"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(const shape& out, const std::vector<argument>& args) const;
};

struct identity
{
    std::string name() const { return "identity"; }
    shape compute_shape(const std::vector<shape>& inputs) const { return inputs.at(0); }
    argument compute(const shape&, const std::vector<argument>& args) const { return args.at(0); }
    std::ptrdiff_t output_alias(const std::vector<shape>&) const { return 0; }
};

// src/include/migraphx/op/capture.hpp:44-77: passes its input through and hands it to a callback;
// inserted by capture_arguments_pass for calibration.
struct capture
{
    std::size_t ins_index = 0;
    std::function<void(std::size_t, std::vector<argument>)> f;
    template <class Self, class F>
    static void reflect(Self& self, F fn)
    {
        fn(self.ins_index, "ins_index");
    }
    std::string name() const { return "capture"; }
    shape compute_shape(const std::vector<shape>& inputs) const { return inputs.at(0); }
    // takes the context so that compile-time evaluation never folds it away
    argument compute(context&, const shape&, const std::vector<argument>& args) const
    {
        if(not f)
            MIGRAPHX_THROW("CAPTURE: callback function is not callable!");
        f(ins_index, args);
        return args.at(0);
    }
    std::ptrdiff_t output_alias(const std::vector<shape>&) const { return 0; }
};

// src/include/migraphx/op/allocate.hpp: an output buffer of a fixed shape; targets replace it
// with their own allocation operator.
struct allocate
{
    shape s;
    std::string name() const { return "allocate"; }
    shape compute_shape(const std::vector<shape>&) const { return s; }
};

} // namespace op
} // namespace migraphx
#endif
