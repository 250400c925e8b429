#include <migraphx/ops.hpp>
#include <migraphx/module.hpp>
#include <migraphx/register_op.hpp>
#include <algorithm>
#include <numeric>
#include <set>

namespace migraphx {
namespace op {

namespace {

void check_count(const std::vector<shape>& inputs, const std::string& name, std::size_t lo, std::size_t hi)
{
    if(inputs.size() < lo or inputs.size() > hi)
        MIGRAPHX_THROW(name + ": Wrong number of arguments: expected " + std::to_string(lo) +
                       (hi != lo ? " to " + std::to_string(hi) : "") + " but given " +
                       std::to_string(inputs.size()));
}

void check_same_dims(const std::vector<shape>& inputs, const std::string& name)
{
    for(const auto& s : inputs)
    {
        if(s.lens() != inputs.front().lens())
            MIGRAPHX_THROW(name + ": Dimensions do not match");
    }
}

int64_t normalize_axis(int64_t axis, std::size_t ndim, const std::string& name)
{
    const auto n = static_cast<int64_t>(ndim);
    if(axis < -n or axis >= n)
        MIGRAPHX_THROW(name + ": axis " + std::to_string(axis) + " out of range for rank " +
                       std::to_string(ndim));
    return axis < 0 ? axis + n : axis;
}

shape same_layout(const shape& in, shape::type_t t, const std::vector<std::size_t>& lens)
{
    if(in.broadcasted() or not in.packed())
        return {t, lens};
    return in.with_lens(t, lens);
}

shape dot_shape(const std::vector<shape>& inputs, const std::string& name, shape::type_t out_type)
{
    const shape& a = inputs.at(0);
    const shape& b = inputs.at(1);
    if(a.type() != b.type())
        MIGRAPHX_THROW(name + ": Types do not match");
    if(a.ndim() != b.ndim())
        MIGRAPHX_THROW(name + ": Number of dimensions do not match");
    if(a.ndim() < 2)
        MIGRAPHX_THROW(name + ": dot only accepts >= 2D operands");
    const std::size_t nd = a.ndim();
    if(not std::equal(a.lens().begin(), a.lens().end() - 2, b.lens().begin()))
        MIGRAPHX_THROW(name + ": outer dimensions of A and B mismatch");
    if(a.lens()[nd - 1] != b.lens()[nd - 2])
        MIGRAPHX_THROW(name + ": inner dimensions are not compatible");
    auto lens    = a.lens();
    lens[nd - 1] = b.lens()[nd - 1];
    return {out_type, lens};
}

} // namespace

shape quant_dot::compute_shape(const std::vector<shape>& inputs) const
{
    if(inputs.size() != 2 and inputs.size() != 4)
        MIGRAPHX_THROW("QUANT_DOT: Wrong number of arguments: expected 2 or 4 but given " +
                       std::to_string(inputs.size()));
    if(inputs.size() == 4 and inputs[2].type() != inputs[3].type())
        MIGRAPHX_THROW("QUANT_DOT: Types do not match");
    const auto t = inputs[0].type();
    static const std::set<shape::type_t> fp8 = {shape::fp8e4m3fn_type,
                                                shape::fp8e4m3fnuz_type,
                                                shape::fp8e5m2_type,
                                                shape::fp8e5m2fnuz_type};
    if(fp8.count(t) == 0 and t != shape::int8_type and t != shape::uint8_type and
       t != shape::float_type)
        MIGRAPHX_THROW("QUANT_DOT: only supports int8_t, uint8_t, float, and fp8");
    const auto out_type =
        (inputs.size() == 4 or fp8.count(t) > 0) ? shape::float_type : shape::int32_type;
    return dot_shape(inputs, "QUANT_DOT", out_type);
}

shape dot::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "DOT", 2, 2);
    return dot_shape(inputs, "DOT", inputs[0].type());
}

std::size_t convolution_attributes::kdims() const
{
    if((padding.size() != stride.size() and padding.size() / 2 != stride.size()) or
       stride.size() != dilation.size())
        MIGRAPHX_THROW("CONVOLUTION: inconsistent attribute sizes");
    return stride.size();
}

std::vector<std::size_t> convolution_attributes::output_lens(const std::string& opname,
                                                             const shape& input,
                                                             const shape& weights) const
{
    if(input.ndim() != weights.ndim() or input.ndim() < 3)
        MIGRAPHX_THROW(opname + ": input and weights need the same rank of at least 3");
    const std::size_t kd = input.ndim() - 2;
    if(kd != kdims())
        MIGRAPHX_THROW(opname + ": input k-dims does not match attribute size");
    if(group < 1 or input.lens()[1] != weights.lens()[1] * static_cast<std::size_t>(group) or
       weights.lens()[0] % static_cast<std::size_t>(group) != 0)
        MIGRAPHX_THROW(opname + ": mismatched channel numbers");
    std::vector<std::size_t> lens{input.lens()[0], weights.lens()[0]};
    for(std::size_t i = 0; i < kd; i++)
    {
        auto padding_factor = 2 * padding[i];
        if(padding.size() == 2 * kd)
            padding_factor = padding[i] + padding[i + kd];
        const auto span = static_cast<std::ptrdiff_t>(input.lens()[i + 2]) -
                          (1 + dilation[i] * (static_cast<std::ptrdiff_t>(weights.lens()[i + 2]) - 1)) +
                          padding_factor;
        // the quotient truncates toward zero, as the reference's signed division does
        lens.push_back(static_cast<std::size_t>(std::max<std::ptrdiff_t>(1, span / stride[i] + 1)));
    }
    return lens;
}

shape convolution::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "CONVOLUTION", 2, 2);
    if(inputs[0].type() != inputs[1].type())
        MIGRAPHX_THROW("CONVOLUTION: Types do not match");
    return {inputs[0].type(), output_lens("CONVOLUTION", inputs[0], inputs[1])};
}

shape quant_convolution::compute_shape(const std::vector<shape>& inputs) const
{
    if(inputs.size() != 2 and inputs.size() != 4)
        MIGRAPHX_THROW("QUANT_CONVOLUTION: Wrong number of arguments: expected 2 or 4 but given " +
                       std::to_string(inputs.size()));
    if(inputs[0].type() != inputs[1].type())
        MIGRAPHX_THROW("QUANT_CONVOLUTION: Types do not match");
    if(inputs.size() == 4 and inputs[2].type() != inputs[3].type())
        MIGRAPHX_THROW("QUANT_CONVOLUTION: Types do not match");
    const auto t = inputs[0].type();
    static const std::set<shape::type_t> fp8 = {shape::fp8e4m3fn_type,
                                                shape::fp8e4m3fnuz_type,
                                                shape::fp8e5m2_type,
                                                shape::fp8e5m2fnuz_type};
    if(fp8.count(t) == 0 and t != shape::int8_type and t != shape::float_type and t != shape::fp4x2_type)
        MIGRAPHX_THROW("QUANT_CONVOLUTION: only supports int8_t, uint8_t, fp4x2, and fp8");
    return {t == shape::int8_type ? shape::int32_type : shape::float_type,
            output_lens("QUANT_CONVOLUTION", inputs[0], inputs[1])};
}

shape quantizelinear::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "QUANTIZELINEAR", 2, 3);
    check_same_dims(inputs, "QUANTIZELINEAR");
    if(inputs[0].type() != inputs[1].type())
        MIGRAPHX_THROW("QUANTIZELINEAR: Scales and input must be the same type");
    if(inputs.size() == 3)
        return same_layout(inputs[0], inputs[2].type(), inputs[0].lens());
    return same_layout(inputs[0],
                       out_type < 0 ? shape::uint8_type : static_cast<shape::type_t>(out_type),
                       inputs[0].lens());
}

shape dequantizelinear::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "DEQUANTIZELINEAR", 2, 3);
    check_same_dims(inputs, "DEQUANTIZELINEAR");
    if(inputs.size() == 3 and inputs[0].type() != inputs[2].type())
        MIGRAPHX_THROW("DEQUANTIZELINEAR: Zero point and input should be the same type.");
    return same_layout(inputs[0], inputs[1].type(), inputs[0].lens());
}

shape unpack_int4::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "UNPACK_INT4", 1, 1);
    const auto& in = inputs[0];
    if(in.type() != shape::int8_type and in.type() != shape::uint8_type)
        MIGRAPHX_THROW("UNPACK_INT4: Only Int8 or Uint8 is supported for unpacking");
    auto lens = in.lens();
    lens[normalize_axis(axis, in.ndim(), "UNPACK_INT4")] *= 2;
    return {in.type(), lens};
}

shape pack_int4::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "PACK_INT4", 1, 1);
    const auto& in = inputs[0];
    if(in.type() != shape::int8_type and in.type() != shape::uint8_type)
        MIGRAPHX_THROW("PACK_INT4: Only Int8 or Uint8 is supported for packing");
    auto lens     = in.lens();
    const auto ax = normalize_axis(axis, in.ndim(), "PACK_INT4");
    if(lens[ax] % 2 != 0)
        MIGRAPHX_THROW("PACK_INT4: Can not pack axis that has odd lengths");
    lens[ax] /= 2;
    return {in.type(), lens};
}

shape unpack_fp4::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "UNPACK_FP4", 1, 1);
    const auto& in = inputs[0];
    if(in.type() != shape::fp4x2_type)
        MIGRAPHX_THROW("UNPACK_FP4: Only fp4x2_type is supported for unpacking");
    auto lens = in.lens();
    lens[normalize_axis(axis, in.ndim(), "UNPACK_FP4")] *= 2;
    return {shape::fp8e4m3fn_type, lens};
}

shape pack_fp4::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "PACK_FP4", 1, 1);
    const auto& in = inputs[0];
    auto lens      = in.lens();
    const auto ax  = normalize_axis(axis, in.ndim(), "PACK_FP4");
    if(lens[ax] % 2 != 0)
        MIGRAPHX_THROW("PACK_FP4: Can not pack along axis of odd length (" + std::to_string(lens[ax]) + ")");
    lens[ax] /= 2;
    return {shape::fp4x2_type, lens};
}

shape convert::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "CONVERT", 1, 1);
    const auto& in = inputs[0];
    // a broadcast or transposed input keeps its strides (op/convert.hpp:52-61)
    if(in.scalar() or in.broadcasted() or in.packed())
        return in.with_type(target_type);
    return {target_type, in.lens()};
}

shape binary::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, op_name, 2, 2);
    if(inputs[0].type() != inputs[1].type())
        MIGRAPHX_THROW(op_name + ": Types do not match");
    check_same_dims(inputs, op_name);
    const auto& s0 = inputs[0];
    const auto& s1 = inputs[1];
    if(s0 == s1 and s0.packed())
        return s0;
    if(s0.packed() != s1.packed())
        return s0.packed() ? s0 : s1;
    if(s0.broadcasted() != s1.broadcasted())
        return s0.broadcasted() ? s1.with_lens(s0.lens()) : s0.with_lens(s0.lens());
    return {s0.type(), s0.lens()};
}

shape unary::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, op_name, 1, 1);
    const auto& s = inputs[0];
    if(s.scalar() or s.broadcasted() or s.packed())
        return s;
    return {s.type(), s.lens()};
}

shape reduce_mean::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "REDUCE_MEAN", 1, 1);
    const auto& s = inputs[0];
    auto lens     = s.lens();
    if(axes.empty())
        std::fill(lens.begin(), lens.end(), 1);
    for(auto a : axes)
        lens[normalize_axis(a, s.ndim(), "REDUCE_MEAN")] = 1;
    return {s.type(), lens};
}

shape reduce_extreme::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, op_name, 1, 1);
    const auto& s = inputs[0];
    auto lens     = s.lens();
    if(axes.empty())
        std::fill(lens.begin(), lens.end(), 1);
    for(auto a : axes)
        lens[normalize_axis(a, s.ndim(), op_name)] = 1;
    return {s.type(), lens};
}

shape clip::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "clip", 3, 3);
    if(inputs[0].type() != inputs[1].type() or inputs[0].type() != inputs[2].type())
        MIGRAPHX_THROW("clip: Types do not match");
    check_same_dims(inputs, "clip");
    return {inputs[0].type(), inputs[0].lens()};
}

shape softmax::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "SOFTMAX", 1, 1);
    const auto& s = inputs[0];
    normalize_axis(axis, s.ndim(), "SOFTMAX");
    if(s.broadcasted())
        return {s.type(), s.lens()};
    return s.packed() ? s.with_lens(s.lens()) : shape{s.type(), s.lens()};
}

shape gather::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "GATHER", 2, 2);
    const auto& data = inputs[0];
    const auto& idx  = inputs[1];
    const auto ax    = normalize_axis(axis, data.ndim(), "GATHER");
    auto lens        = data.lens();
    lens.erase(lens.begin() + ax);
    const bool scalar_indices = idx.ndim() == 1 and idx.scalar() and idx.elements() == 1;
    if(not scalar_indices)
        lens.insert(lens.begin() + ax, idx.lens().begin(), idx.lens().end());
    if(lens.empty())
        return shape{data.type()};
    return {data.type(), lens};
}

shape broadcast::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "BROADCAST", 1, 1);
    const auto& in = inputs[0];
    if(axis >= out_lens.size())
        MIGRAPHX_THROW("BROADCAST : axis " + std::to_string(axis) + " is out of range");
    if(out_lens.size() - axis < in.ndim())
        MIGRAPHX_THROW("BROADCAST: (broadcast ndims - axis) is less than input ndims");
    std::vector<std::size_t> strides(out_lens.size(), 0);
    for(std::size_t i = 0; i < in.ndim(); i++)
    {
        if(in.lens()[i] != out_lens[axis + i] and in.lens()[i] != 1)
            MIGRAPHX_THROW("BROADCAST: input and output dimensions do not match at axis " +
                           std::to_string(axis + i));
        strides[axis + i] = in.lens()[i] == 1 ? 0 : in.strides()[i];
    }
    return {in.type(), out_lens, strides};
}

shape multibroadcast::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "MULTIBROADCAST", 1, 1);
    const auto& in = inputs[0];
    if(in.ndim() == 0)
        MIGRAPHX_THROW("MULTIBROADCAST: input dimensions should be > 0");
    if(in.ndim() > out_lens.size())
        MIGRAPHX_THROW("MULTIBROADCAST: input dimensions should <= output size");
    const std::size_t offset = out_lens.size() - in.ndim();
    std::vector<std::size_t> strides(out_lens.size(), 0);
    for(std::size_t i = 0; i < in.ndim(); i++)
    {
        if(in.lens()[i] != out_lens[offset + i] and in.lens()[i] != 1)
            MIGRAPHX_THROW("MULTIBROADCAST: input shape cannot be broadcast to the output lens");
        strides[offset + i] = in.lens()[i] == 1 ? 0 : in.strides()[i];
    }
    return {in.type(), out_lens, strides};
}

shape transpose::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "TRANSPOSE", 1, 1);
    const auto& in = inputs[0];
    if(permutation.size() != in.ndim())
        MIGRAPHX_THROW("TRANSPOSE: Permutation has wrong number of axes");
    std::vector<int64_t> sorted = permutation;
    std::sort(sorted.begin(), sorted.end());
    for(std::size_t i = 0; i < sorted.size(); i++)
    {
        if(sorted[i] != static_cast<int64_t>(i))
            MIGRAPHX_THROW("TRANSPOSE: Invalid permutation");
    }
    std::vector<std::size_t> lens(in.ndim());
    std::vector<std::size_t> strides(in.ndim());
    for(std::size_t i = 0; i < in.ndim(); i++)
    {
        lens[i]    = in.lens()[permutation[i]];
        strides[i] = in.strides()[permutation[i]];
    }
    return {in.type(), lens, strides};
}

shape reshape::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "RESHAPE", 1, 1);
    const auto& in = inputs[0];
    std::vector<std::size_t> lens(dims.size());
    int64_t infer     = -1;
    std::size_t known = 1;
    for(std::size_t i = 0; i < dims.size(); i++)
    {
        if(dims[i] == -1)
        {
            if(infer >= 0)
                MIGRAPHX_THROW("RESHAPE: Dimensions do not match");
            infer = static_cast<int64_t>(i);
            continue;
        }
        if(dims[i] == 0)
        {
            if(i >= in.ndim())
                MIGRAPHX_THROW("RESHAPE: 0 dimension beyond the input rank");
            lens[i] = in.lens()[i];
        }
        else if(dims[i] < 0)
            MIGRAPHX_THROW("RESHAPE: negative dimension");
        else
            lens[i] = static_cast<std::size_t>(dims[i]);
        known *= lens[i];
    }
    if(infer >= 0)
    {
        if(known == 0 or in.elements() % known != 0)
            MIGRAPHX_THROW("RESHAPE: Wrong number of elements for reshape");
        lens[infer] = in.elements() / known;
    }
    shape out{in.type(), lens};
    if(out.elements() != in.elements())
        MIGRAPHX_THROW("RESHAPE: Wrong number of elements for reshape: reshape has " +
                       std::to_string(out.elements()) + " elements whereas the input has " +
                       std::to_string(in.elements()));
    return out;
}

argument reshape::compute(const shape& out, const std::vector<argument>& args) const
{
    const auto& in = args.at(0);
    if(in.get_shape().standard())
        return in.reshape(out);
    return contiguous{}.compute(shape{out.type(), in.get_shape().lens()}, args).reshape(out);
}

shape unsqueeze::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "UNSQUEEZE", 1, 1);
    const auto& in         = inputs[0];
    const std::size_t rank = in.ndim() + axes.size();
    std::set<int64_t> ax;
    for(auto a : axes)
        ax.insert(normalize_axis(a, rank, "UNSQUEEZE"));
    if(ax.size() != axes.size())
        MIGRAPHX_THROW("UNSQUEEZE: Axis dimension is not unique");
    if(in.scalar() and in.elements() == 1 and in.ndim() == 1)
        return {in.type(), std::vector<std::size_t>(axes.size(), 1), std::vector<std::size_t>(axes.size(), 0)};
    std::vector<std::size_t> lens(rank);
    std::vector<std::size_t> strides(rank);
    std::size_t p = 0;
    for(std::size_t i = 0; i < rank; i++)
    {
        if(ax.count(static_cast<int64_t>(i)) > 0)
        {
            lens[i] = 1;
            // stride that keeps a standard tensor standard: that of the next input dimension
            // times its length, or 1 past the end
            strides[i] = p < in.ndim() ? in.strides()[p] * in.lens()[p] : 1;
        }
        else
        {
            lens[i]    = in.lens()[p];
            strides[i] = in.strides()[p];
            p++;
        }
    }
    return {in.type(), lens, strides};
}

shape squeeze::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "SQUEEZE", 1, 1);
    const auto& in = inputs[0];
    std::set<int64_t> ax;
    for(auto a : axes)
        ax.insert(normalize_axis(a, in.ndim(), "SQUEEZE"));
    for(auto a : ax)
    {
        if(in.lens()[a] != 1)
            MIGRAPHX_THROW("SQUEEZE: axis dimension is not equal to 1");
    }
    std::vector<std::size_t> lens;
    std::vector<std::size_t> strides;
    for(std::size_t i = 0; i < in.ndim(); i++)
    {
        const bool drop = axes.empty() ? in.lens()[i] == 1 : ax.count(static_cast<int64_t>(i)) > 0;
        if(drop)
            continue;
        lens.push_back(in.lens()[i]);
        strides.push_back(in.strides()[i]);
    }
    if(lens.empty())
        return shape{in.type()};
    return {in.type(), lens, strides};
}

shape slice::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "SLICE", 1, 1);
    const auto& in = inputs[0];
    if(starts.size() != axes.size() or ends.size() != axes.size())
        MIGRAPHX_THROW("SLICE: starts, ends and axes differ in length");
    auto lens = in.lens();
    for(std::size_t i = 0; i < axes.size(); i++)
    {
        const auto ax = normalize_axis(axes[i], in.ndim(), "SLICE");
        const auto n  = static_cast<int64_t>(in.lens()[ax]);
        auto clampi   = [&](int64_t v) { return std::max<int64_t>(0, std::min<int64_t>(n, v < 0 ? v + n : v)); };
        const auto s  = clampi(starts[i]);
        const auto e  = clampi(ends[i]);
        if(e < s)
            MIGRAPHX_THROW("SLICE: end before start");
        lens[ax] = static_cast<std::size_t>(e - s);
    }
    return {in.type(), lens, in.strides()};
}

std::size_t slice::compute_offset(const shape& in) const
{
    std::size_t off = 0;
    for(std::size_t i = 0; i < axes.size(); i++)
    {
        const auto ax = normalize_axis(axes[i], in.ndim(), "SLICE");
        const auto n  = static_cast<int64_t>(in.lens()[ax]);
        const auto s  = std::max<int64_t>(0, std::min<int64_t>(n, starts[i] < 0 ? starts[i] + n : starts[i]));
        off += static_cast<std::size_t>(s) * in.strides()[ax];
    }
    return off;
}

shape contiguous::compute_shape(const std::vector<shape>& inputs) const
{
    check_count(inputs, "CONTIGUOUS", 1, 1);
    return {inputs[0].type(), inputs[0].lens()};
}

argument contiguous::compute(const shape& out, const std::vector<argument>& args) const
{
    const auto& in      = args.at(0);
    const auto& s       = in.get_shape();
    const std::size_t w = s.type_size();
    argument r{out};
    const std::size_t n = s.elements();
    for(std::size_t i = 0; i < n; i++)
        std::memcpy(r.data() + i * w, in.data() + s.index(i) * w, w);
    return r;
}

} // namespace op

MIGRAPHX_REGISTER_OP(op::quant_dot);
MIGRAPHX_REGISTER_OP(op::dot);
MIGRAPHX_REGISTER_OP(op::convolution);
MIGRAPHX_REGISTER_OP(op::quant_convolution);
MIGRAPHX_REGISTER_OP(op::quantizelinear);
MIGRAPHX_REGISTER_OP(op::dequantizelinear);
MIGRAPHX_REGISTER_OP(op::unpack_int4);
MIGRAPHX_REGISTER_OP(op::unpack_fp4);
MIGRAPHX_REGISTER_OP(op::pack_fp4);
MIGRAPHX_REGISTER_OP(op::pack_int4);
MIGRAPHX_REGISTER_OP(op::convert);
MIGRAPHX_REGISTER_OP(op::mul);
MIGRAPHX_REGISTER_OP(op::add);
MIGRAPHX_REGISTER_OP(op::sub);
MIGRAPHX_REGISTER_OP(op::div);
MIGRAPHX_REGISTER_OP(op::max);
MIGRAPHX_REGISTER_OP(op::min);
MIGRAPHX_REGISTER_OP(op::nearbyint);
MIGRAPHX_REGISTER_OP(op::reduce_max);
MIGRAPHX_REGISTER_OP(op::reduce_min);
MIGRAPHX_REGISTER_OP(op::clip);
MIGRAPHX_REGISTER_OP(op::erf);
MIGRAPHX_REGISTER_OP(op::sqrt);
MIGRAPHX_REGISTER_OP(op::rsqrt);
MIGRAPHX_REGISTER_OP(op::exp);
MIGRAPHX_REGISTER_OP(op::tanh);
MIGRAPHX_REGISTER_OP(op::neg);
MIGRAPHX_REGISTER_OP(op::reduce_mean);
MIGRAPHX_REGISTER_OP(op::softmax);
MIGRAPHX_REGISTER_OP(op::gather);
MIGRAPHX_REGISTER_OP(op::broadcast);
MIGRAPHX_REGISTER_OP(op::multibroadcast);
MIGRAPHX_REGISTER_OP(op::transpose);
MIGRAPHX_REGISTER_OP(op::reshape);
MIGRAPHX_REGISTER_OP(op::unsqueeze);
MIGRAPHX_REGISTER_OP(op::squeeze);
MIGRAPHX_REGISTER_OP(op::slice);
MIGRAPHX_REGISTER_OP(op::contiguous);
MIGRAPHX_REGISTER_OP(op::identity);
MIGRAPHX_REGISTER_OP(op::capture);
MIGRAPHX_REGISTER_OP(op::allocate);
MIGRAPHX_REGISTER_OP(builtin::literal_op);
MIGRAPHX_REGISTER_OP(builtin::param);
MIGRAPHX_REGISTER_OP(builtin::returns);

} // namespace migraphx
