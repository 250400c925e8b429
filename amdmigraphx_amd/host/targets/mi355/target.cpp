#include "device_ops.hpp"
#include <migraphx/ops.hpp>
#include <migraphx/passes.hpp>
#include <migraphx/register_op.hpp>
#include <cstdlib>
#include <migraphx/register_target.hpp>
#include <hip/hip_runtime_api.h>
#include <algorithm>

namespace migraphx {
namespace mi355 {

namespace {

void hip_check(hipError_t e, const char* what)
{
    if(e != hipSuccess)
        MIGRAPHX_THROW(std::string("mi355: ") + what + " failed: " + hipGetErrorString(e));
}

void status_check(int st, const std::string& what)
{
    if(st != MI355_OK)
        MIGRAPHX_THROW(what + ": " + mi355_status_string(st));
}

void* stream_of(migraphx::context& ctx) { return any_cast<context>(ctx).get_stream(); }

void check_inputs(const std::vector<shape>& inputs, std::size_t n, const std::string& name)
{
    if(inputs.size() != n)
        MIGRAPHX_THROW(name + ": expected " + std::to_string(n) + " arguments, got " +
                       std::to_string(inputs.size()));
}

void check_standard(const shape& s, const std::string& name)
{
    if(not s.standard())
        MIGRAPHX_THROW(name + ": tensor must be in standard layout");
}

} // namespace

// ----------------------------------------------------------------- context, memory

struct context::stream_holder
{
    hipStream_t s = nullptr;
    stream_holder() { hip_check(hipStreamCreate(&s), "hipStreamCreate"); }
    stream_holder(const stream_holder&) = delete;
    stream_holder& operator=(const stream_holder&) = delete;
    ~stream_holder()
    {
        if(s != nullptr)
            (void)hipStreamDestroy(s);
    }
};

context::context() : m_stream(std::make_shared<stream_holder>()) {}
void* context::get_stream() const { return m_stream->s; }
void context::finish() const { hip_check(hipStreamSynchronize(m_stream->s), "hipStreamSynchronize"); }

argument allocate_device(const shape& s)
{
    void* p             = nullptr;
    const std::size_t n = std::max<std::size_t>(s.bytes(), 16);
    hip_check(hipMalloc(&p, n), "hipMalloc");
    return {s, std::shared_ptr<char>(static_cast<char*>(p), [](char* q) { (void)hipFree(q); })};
}

argument to_device(const argument& host)
{
    // the device copy is dense in the host tensor's own memory order: same shape, same strides
    argument d = allocate_device(host.get_shape());
    if(host.get_shape().bytes() > 0)
        hip_check(hipMemcpy(d.data(), host.data(), host.get_shape().bytes(), hipMemcpyHostToDevice),
                  "hipMemcpy to device");
    return d;
}

argument from_device(const argument& device)
{
    argument h{device.get_shape()};
    if(device.get_shape().bytes() > 0)
        hip_check(
            hipMemcpy(h.data(), device.data(), device.get_shape().bytes(), hipMemcpyDeviceToHost),
            "hipMemcpy from device");
    return h;
}

// ----------------------------------------------------------------- helpers

int to_mi355_type(shape::type_t t)
{
    switch(t)
    {
    case shape::int8_type: return MI355_I8;
    case shape::uint8_type: return MI355_U8;
    case shape::int32_type: return MI355_I32;
    case shape::float_type: return MI355_F32;
    case shape::half_type: return MI355_F16;
    case shape::bf16_type: return MI355_BF16;
    case shape::fp8e4m3fn_type: return MI355_FP8;
    case shape::fp8e5m2_type: return MI355_BF8;
    default: MIGRAPHX_THROW("mi355: no kernel takes " + shape::type_name(t));
    }
}

matrix_view view_as_matrix(const shape& s)
{
    matrix_view v;
    const std::size_t nd = s.ndim();
    if(nd < 2)
        return v;
    v.rows     = static_cast<int64_t>(s.lens()[nd - 2]);
    v.cols     = static_cast<int64_t>(s.lens()[nd - 1]);
    v.stride_r = v.rows == 1 ? 0 : static_cast<int64_t>(s.strides()[nd - 2]);
    v.stride_c = v.cols == 1 ? 0 : static_cast<int64_t>(s.strides()[nd - 1]);
    if(v.cols == 1 or v.stride_c == 1)
    {
        v.trans = false;
        v.ld    = v.rows == 1 ? v.cols : v.stride_r;
        v.ok    = v.ld >= v.cols;
    }
    else if(v.rows == 1 or v.stride_r == 1)
    {
        v.trans = true;
        v.ld    = v.stride_c;
        v.ok    = v.ld >= v.rows;
    }
    if(not v.ok)
        return v;
    // leading dimensions must collapse into one batch stride
    std::vector<std::pair<std::size_t, std::size_t>> dims; // (len, stride), length-1 dims dropped
    for(std::size_t i = 0; i + 2 < nd; i++)
    {
        v.batch *= static_cast<int64_t>(s.lens()[i]);
        if(s.lens()[i] > 1)
            dims.emplace_back(s.lens()[i], s.strides()[i]);
    }
    for(std::size_t i = 0; i + 1 < dims.size(); i++)
    {
        if(dims[i].second != dims[i + 1].second * dims[i + 1].first)
            v.ok = false;
    }
    v.batch_stride = dims.empty() ? 0 : static_cast<int64_t>(dims.back().second);
    return v;
}

bool collapse_2d(const shape& s, int64_t& stride_r, int64_t& stride_c)
{
    const std::size_t nd = s.ndim();
    if(nd == 0)
        return false;
    stride_c = s.lens()[nd - 1] == 1 ? 0 : static_cast<int64_t>(s.strides()[nd - 1]);
    std::vector<std::pair<std::size_t, std::size_t>> dims;
    for(std::size_t i = 0; i + 1 < nd; i++)
    {
        if(s.lens()[i] > 1)
            dims.emplace_back(s.lens()[i], s.strides()[i]);
    }
    for(std::size_t i = 0; i + 1 < dims.size(); i++)
    {
        if(dims[i].second != dims[i + 1].second * dims[i + 1].first)
            return false;
    }
    stride_r = dims.empty() ? 0 : static_cast<int64_t>(dims.back().second);
    return true;
}

bool batch_collapses(const shape& s)
{
    if(s.ndim() <= 3)
        return true;
    std::vector<std::size_t> bl(s.lens().begin(), s.lens().end() - 2);
    std::vector<std::size_t> bs(s.strides().begin(), s.strides().end() - 2);
    bl.push_back(1);
    bs.push_back(1);
    int64_t sr = 0;
    int64_t sc = 0;
    return collapse_2d(shape{s.type(), bl, bs}, sr, sc);
}

namespace {
void rows_cols(const shape& s, int64_t& rows, int64_t& cols)
{
    cols = static_cast<int64_t>(s.lens().back());
    rows = cols == 0 ? 0 : static_cast<int64_t>(s.elements()) / cols;
}
} // namespace

// ----------------------------------------------------------------- memory operators

argument allocate::compute(migraphx::context&, const shape&, const std::vector<argument>&) const
{
    if(buffer.empty())
        MIGRAPHX_THROW("mi355::allocate: evaluated before finalize");
    return buffer;
}

argument arena::compute(migraphx::context&, const shape&, const std::vector<argument>&) const
{
    if(buffer.empty())
        MIGRAPHX_THROW("mi355::arena: evaluated before finalize");
    return buffer;
}

shape load::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 1, name());
    if(offset + s.bytes() > inputs.front().bytes())
        MIGRAPHX_THROW("mi355::load: reaches past the end of the arena");
    return s;
}

value device_literal::to_value() const
{
    // the key is always there: make_op checks attribute names against a default instance
    value v   = value::object();
    v["data"] = value("data", data.empty() ? value{} : migraphx::to_value(from_device(data)));
    return v;
}

void device_literal::from_value(const value& v)
{
    if(not v.contains("data") or v.at("data").is_null())
        return;
    data = to_device(migraphx::from_value<argument>(v.at("data")));
}

shape copy_to_device::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    if(inputs[0] != inputs[1])
        MIGRAPHX_THROW("mi355::copy_to_device: host and device shapes differ");
    return inputs[1];
}

argument copy_to_device::compute(migraphx::context& ctx,
                                 const shape&,
                                 const std::vector<argument>& args) const
{
    const auto n = args[0].get_shape().bytes();
    if(n > 0)
        hip_check(hipMemcpyAsync(args[1].data(),
                                 args[0].data(),
                                 n,
                                 hipMemcpyHostToDevice,
                                 static_cast<hipStream_t>(stream_of(ctx))),
                  "hipMemcpyAsync to device");
    return args[1];
}

shape copy_from_device::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 1, name());
    return inputs[0];
}

argument copy_from_device::compute(migraphx::context& ctx,
                                   const shape& out,
                                   const std::vector<argument>& args) const
{
    argument h{out};
    auto s = static_cast<hipStream_t>(stream_of(ctx));
    if(out.bytes() > 0)
        hip_check(hipMemcpyAsync(h.data(), args[0].data(), out.bytes(), hipMemcpyDeviceToHost, s),
                  "hipMemcpyAsync from device");
    hip_check(hipStreamSynchronize(s), "hipStreamSynchronize");
    return h;
}

// ----------------------------------------------------------------- GEMM operators

shape quant_dot::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, expected_inputs(), name());
    auto s = op::quant_dot{}.compute_shape({inputs[0], inputs[1]});
    const bool bare_u8 = inputs[0].type() == shape::uint8_type and not dequant;
    if(inputs[0].type() != shape::int8_type and inputs[0].type() != shape::fp8e4m3fn_type and
       inputs[0].type() != shape::fp8e5m2_type and not bare_u8)
        MIGRAPHX_THROW("mi355::quant_dot: kernels take int8, fp8e4m3fn or fp8e5m2 operands (uint8 for the "
                       "bare result), not " + inputs[0].type_string());
    if(not view_as_matrix(inputs[0]).ok or not view_as_matrix(inputs[1]).ok)
        MIGRAPHX_THROW("mi355::quant_dot: operand strides are neither row-major nor transposed");
    if(not dequant and out_type != s.type())
        MIGRAPHX_THROW("mi355::quant_dot: output type must be " + s.type_string());
    if(dequant)
    {
        if(out_type != shape::float_type and out_type != shape::half_type and
           out_type != shape::bf16_type)
            MIGRAPHX_THROW("mi355::quant_dot: dequantized output must be float, half or bf16");
        if(inputs[2].type() != shape::float_type or inputs[3].type() != shape::float_type)
            MIGRAPHX_THROW("mi355::quant_dot: scales must be float");
        if((zp_a != 0 or zp_b != 0) and inputs[0].type() != shape::int8_type)
            MIGRAPHX_THROW("mi355::quant_dot: zero points need int8 operands");
    }
    if(workspace and inputs[inputs.size() - 2].type() != shape::uint8_type)
        MIGRAPHX_THROW("mi355::quant_dot: the workspace must be a uint8 buffer");
    if(has_bias)
    {
        const shape& bias = inputs[inputs.size() - (workspace ? 3 : 2)];
        if(not dequant)
            MIGRAPHX_THROW("mi355::quant_dot: a bias needs the dequantizing epilogue");
        const auto per = scale_b_mode == MI355_QP_PER_COL_BATCH ? s.elements() / s.lens()[s.ndim() - 2] : s.lens().back();
        if(bias.type() != shape::float_type or not bias.standard() or bias.elements() != per)
            MIGRAPHX_THROW("mi355::quant_dot: the bias must be a dense float vector of N elements (one per batch "
                           "entry with column scales per batch entry)");
    }
    if(scale_b_mode == MI355_QP_PER_COL_BATCH)
    {
        // [batch, N]: one vector of column scales per batch entry
        if(not dequant or not inputs[3].standard() or
           inputs[3].elements() != s.elements() / s.lens()[s.ndim() - 2])
            MIGRAPHX_THROW("mi355::quant_dot: column scales per batch entry are a dense [batch, N] tensor");
    }
    shape out{out_type, s.lens()};
    if(inputs.back() != out)
        MIGRAPHX_THROW("mi355::quant_dot: output buffer has the wrong shape");
    return out;
}

mi355_quant_dot_desc quant_dot::describe(const shape& a, const shape& b) const
{
    const auto va = view_as_matrix(a);
    const auto vb = view_as_matrix(b);
    mi355_quant_dot_desc d{};
    d.m        = va.rows;
    d.k        = va.cols;
    d.n        = vb.cols;
    d.trans_a  = va.trans;
    d.trans_b  = vb.trans;
    d.lda      = va.ld;
    d.ldb      = vb.ld;
    d.ldc      = d.n;
    d.batch    = va.batch;
    d.stride_a = va.batch_stride;
    d.stride_b = vb.batch_stride;
    d.stride_c = d.m * d.n;
    d.in_type  = to_mi355_type(a.type());
    d.out_type = to_mi355_type(out_type);
    d.dequant  = dequant ? 1 : 0;
    d.scale_a_mode = static_cast<int32_t>(scale_a_mode);
    d.scale_b_mode = static_cast<int32_t>(scale_b_mode);
    d.zp_a         = static_cast<int32_t>(zp_a);
    d.zp_b         = static_cast<int32_t>(zp_b);
    return d;
}

argument quant_dot::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const auto d     = describe(args[0].get_shape(), args[1].get_shape());
    std::size_t next = 2;
    const float* sa  = nullptr;
    const float* sb  = nullptr;
    if(dequant)
    {
        sa = reinterpret_cast<const float*>(args[next++].data());
        sb = reinterpret_cast<const float*>(args[next++].data());
    }
    const int32_t* colsum_b = zp_a != 0 ? reinterpret_cast<const int32_t*>(args[next++].data()) : nullptr;
    const int32_t* rowsum_a = zp_b != 0 ? reinterpret_cast<const int32_t*>(args[next++].data()) : nullptr;
    const float* bias = has_bias ? reinterpret_cast<const float*>(args[next++].data()) : nullptr;
    if((zp_a != 0 or zp_b != 0) and d.batch != 1)
        MIGRAPHX_THROW("mi355::quant_dot: zero points with batched operands are not supported");
    void* ws             = workspace ? args[next].data() : nullptr;
    const size_t ws_size = workspace ? args[next].get_shape().bytes() : 0;
    status_check(mi355_quant_dot_ws(&d,
                                    args[0].data(),
                                    args[1].data(),
                                    args.back().data(),
                                    sa,
                                    sb,
                                    colsum_b,
                                    rowsum_a,
                                    bias,
                                    ws,
                                    ws_size,
                                    stream_of(ctx)),
                 name());
    return args.back();
}

shape quant_dot_prepack::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    const shape& b = inputs[0];
    const auto vb  = view_as_matrix(b);
    if(b.ndim() != 2 or not vb.ok)
        MIGRAPHX_THROW("mi355::quant_dot_prepack: B is a row-major or transposed matrix");
    const size_t bytes = mi355_quant_dot_prepacked_size(to_mi355_type(b.type()), vb.cols, vb.rows);
    if(bytes == 0)
        MIGRAPHX_THROW("mi355::quant_dot_prepack: the reordered form does not take this shape");
    shape out{shape::uint8_type, {bytes}};
    if(inputs.back() != out)
        MIGRAPHX_THROW("mi355::quant_dot_prepack: output buffer has the wrong size");
    return out;
}

argument quant_dot_prepack::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const shape& b = args[0].get_shape();
    const auto vb  = view_as_matrix(b);
    status_check(mi355_quant_dot_prepack(args[0].data(),
                                         to_mi355_type(b.type()),
                                         vb.cols,
                                         vb.rows,
                                         vb.trans ? 1 : vb.ld,
                                         vb.trans ? vb.ld : 1,
                                         args.back().data(),
                                         stream_of(ctx)),
                 name());
    return args.back();
}

mi355_quant_dot_desc quant_dot_prepacked::describe(const shape& a, const shape& out) const
{
    mi355_quant_dot_desc d{};
    d.m        = static_cast<int64_t>(a.lens()[0]);
    d.k        = static_cast<int64_t>(a.lens()[1]);
    d.n        = static_cast<int64_t>(out.lens()[1]);
    d.lda      = d.k;
    d.ldb      = d.n;
    d.ldc      = d.n;
    d.batch    = 1;
    d.in_type  = to_mi355_type(a.type());
    d.out_type = to_mi355_type(out_type);
    d.dequant  = dequant ? 1 : 0;
    d.scale_a_mode = static_cast<int32_t>(scale_a_mode);
    d.scale_b_mode = static_cast<int32_t>(scale_b_mode);
    d.zp_a         = static_cast<int32_t>(zp_a);
    d.zp_b         = static_cast<int32_t>(zp_b);
    return d;
}

shape quant_dot_prepacked::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, expected_inputs(), name());
    const shape& a   = inputs[0];
    const shape& out = inputs.back();
    if(a.ndim() != 2 or not a.standard() or out.ndim() != 2 or not out.standard() or out.lens()[0] != a.lens()[0])
        MIGRAPHX_THROW("mi355::quant_dot_prepacked: A and the output are dense matrices with the same rows");
    if(a.lens()[0] > 16)
        MIGRAPHX_THROW("mi355::quant_dot_prepacked: takes at most 16 rows");
    if(inputs[1].type() != shape::uint8_type or
       inputs[1].elements() != mi355_quant_dot_prepacked_size(to_mi355_type(a.type()), out.lens()[1], a.lens()[1]) or
       inputs[1].elements() == 0)
        MIGRAPHX_THROW("mi355::quant_dot_prepacked: the reordered B does not fit the operands");
    const bool fp8 = a.type() != shape::int8_type;
    if(out.type() != out_type or (not dequant and out_type != (fp8 ? shape::float_type : shape::int32_type)))
        MIGRAPHX_THROW("mi355::quant_dot_prepacked: output buffer has the wrong type");
    if(dequant)
    {
        if(out_type != shape::float_type and out_type != shape::half_type and out_type != shape::bf16_type)
            MIGRAPHX_THROW("mi355::quant_dot_prepacked: dequantized output must be float, half or bf16");
        if(inputs[2].type() != shape::float_type or inputs[3].type() != shape::float_type)
            MIGRAPHX_THROW("mi355::quant_dot_prepacked: scales must be float");
        if((zp_a != 0 or zp_b != 0) and fp8)
            MIGRAPHX_THROW("mi355::quant_dot_prepacked: zero points need int8 operands");
    }
    if(has_bias)
    {
        const shape& bias = inputs[inputs.size() - 2];
        if(not dequant or bias.type() != shape::float_type or not bias.standard() or
           bias.elements() != out.lens()[1])
            MIGRAPHX_THROW("mi355::quant_dot_prepacked: the bias is a dense float vector of N elements behind "
                           "the dequantizing epilogue");
    }
    return out;
}

argument
quant_dot_prepacked::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const auto d     = describe(args[0].get_shape(), args.back().get_shape());
    std::size_t next = 2;
    const float* sa  = nullptr;
    const float* sb  = nullptr;
    if(dequant)
    {
        sa = reinterpret_cast<const float*>(args[next++].data());
        sb = reinterpret_cast<const float*>(args[next++].data());
    }
    const int32_t* colsum_b = zp_a != 0 ? reinterpret_cast<const int32_t*>(args[next++].data()) : nullptr;
    const int32_t* rowsum_a = zp_b != 0 ? reinterpret_cast<const int32_t*>(args[next++].data()) : nullptr;
    const float* bias = has_bias ? reinterpret_cast<const float*>(args[next++].data()) : nullptr;
    status_check(mi355_quant_dot_prepacked(
                     &d, args[0].data(), args[1].data(), args.back().data(), sa, sb, colsum_b, rowsum_a, bias, stream_of(ctx)),
                 name());
    return args.back();
}

mi355_quant_conv3d_desc quant_convolution::describe(const shape& x, const shape& w) const
{
    const std::size_t kd = stride.size();
    if(kd < 1 or kd > 3 or dilation.size() != kd or (padding.size() != kd and padding.size() != 2 * kd))
        MIGRAPHX_THROW("mi355::quant_convolution: one to three spatial dimensions with matching attributes");
    if(x.ndim() != kd + 2 or w.ndim() != kd + 2)
        MIGRAPHX_THROW("mi355::quant_convolution: input rank does not match the attributes");
    const bool both_sides = padding.size() == 2 * kd; // low values first, then high values
    const std::size_t lead = 3 - kd;                  // missing leading axes have length one
    mi355_quant_conv3d_desc d{};
    int64_t in[3]  = {1, 1, 1};
    int64_t win[3] = {1, 1, 1};
    for(std::size_t i = 0; i < 3; i++)
    {
        d.stride[i] = 1;
        d.dil[i]    = 1;
    }
    for(std::size_t i = 0; i < kd; i++)
    {
        in[lead + i]       = static_cast<int64_t>(x.lens()[2 + i]);
        win[lead + i]      = static_cast<int64_t>(w.lens()[2 + i]);
        d.pad[lead + i]    = padding[i];
        d.pad_hi[lead + i] = padding[both_sides ? kd + i : i];
        d.stride[lead + i] = stride[i];
        d.dil[lead + i]    = dilation[i];
    }
    d.n = static_cast<int64_t>(x.lens()[0]);
    d.c = static_cast<int64_t>(x.lens()[1]);
    d.o = static_cast<int64_t>(w.lens()[0]);
    d.d = in[0], d.h = in[1], d.w = in[2];
    d.kd = win[0], d.kh = win[1], d.kw = win[2];
    d.group    = group;
    d.in_type  = to_mi355_type(x.type());
    d.out_type = to_mi355_type(out_type);
    d.dequant  = dequant ? 1 : 0;
    d.scale_x_mode = dequant ? MI355_QP_PER_TENSOR : MI355_QP_NONE;
    d.scale_w_mode = dequant ? static_cast<int32_t>(scale_w_mode) : MI355_QP_NONE;
    return d;
}

shape quant_convolution::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, dequant ? 6 : 4, name());
    op::quant_convolution ref;
    ref.padding  = padding;
    ref.stride   = stride;
    ref.dilation = dilation;
    ref.group    = group;
    auto s = ref.compute_shape({inputs[0], inputs[1]});
    if(inputs[0].type() != shape::int8_type and inputs[0].type() != shape::fp8e4m3fn_type)
        MIGRAPHX_THROW("mi355::quant_convolution: kernels take int8 or fp8e4m3fn operands, not " +
                       inputs[0].type_string());
    check_standard(inputs[0], name());
    check_standard(inputs[1], name());
    if(not dequant and out_type != s.type())
        MIGRAPHX_THROW("mi355::quant_convolution: output type must be " + s.type_string());
    if(dequant)
    {
        if(out_type != shape::float_type and out_type != shape::half_type and out_type != shape::bf16_type)
            MIGRAPHX_THROW("mi355::quant_convolution: dequantized output must be float, half or bf16");
        if(inputs[2].type() != shape::float_type or inputs[3].type() != shape::float_type)
            MIGRAPHX_THROW("mi355::quant_convolution: scales must be float");
        if(scale_w_mode != MI355_QP_PER_TENSOR and scale_w_mode != MI355_QP_PER_ROW)
            MIGRAPHX_THROW("mi355::quant_convolution: weight scales are per tensor or per output channel");
    }
    const auto d = describe(inputs[0], inputs[1]);
    size_t need  = 0;
    status_check(mi355_quant_convolution3d_dims(&d, nullptr, &need), name());
    const shape& ws = inputs[inputs.size() - 2];
    if(ws.type() != shape::uint8_type or not ws.standard() or ws.bytes() < need)
        MIGRAPHX_THROW("mi355::quant_convolution: workspace too small");
    shape out{out_type, s.lens()};
    if(inputs.back() != out)
        MIGRAPHX_THROW("mi355::quant_convolution: output buffer has the wrong shape");
    return out;
}

argument
quant_convolution::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const auto d = describe(args[0].get_shape(), args[1].get_shape());
    const float* sx = dequant ? reinterpret_cast<const float*>(args[2].data()) : nullptr;
    const float* sw = dequant ? reinterpret_cast<const float*>(args[3].data()) : nullptr;
    const argument& ws = args[args.size() - 2];
    status_check(mi355_quant_convolution3d(&d,
                                         args[0].data(),
                                         args[1].data(),
                                         args.back().data(),
                                         sx,
                                         sw,
                                         ws.data(),
                                         ws.get_shape().bytes(),
                                         stream_of(ctx)),
                 name());
    return args.back();
}

shape convolution::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 3, name());
    op::convolution ref;
    ref.padding  = padding;
    ref.stride   = stride;
    ref.dilation = dilation;
    ref.group    = group;
    auto s = ref.compute_shape({inputs[0], inputs[1]});
    if(inputs[0].type() != shape::float_type or inputs[1].type() != shape::float_type)
        MIGRAPHX_THROW("mi355::convolution: float tensors only, not " + inputs[0].type_string());
    check_standard(inputs[0], name());
    check_standard(inputs[1], name());
    shape out{shape::float_type, s.lens()};
    if(inputs.back() != out)
        MIGRAPHX_THROW("mi355::convolution: output buffer has the wrong shape");
    return out;
}

argument convolution::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    quant_convolution q;
    q.padding  = padding;
    q.stride   = stride;
    q.dilation = dilation;
    q.group    = group;
    q.out_type = shape::float_type;
    const auto d = q.describe(args[0].get_shape(), args[1].get_shape());
    status_check(mi355_convolution_f32(&d,
                                       reinterpret_cast<const float*>(args[0].data()),
                                       reinterpret_cast<const float*>(args[1].data()),
                                       reinterpret_cast<float*>(args.back().data()),
                                       stream_of(ctx)),
                 name());
    return args.back();
}

shape colsum::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    const auto v = view_as_matrix(inputs[0]);
    if(not v.ok or v.batch != 1 or inputs[0].type() != shape::int8_type)
        MIGRAPHX_THROW("mi355::colsum: needs one int8 matrix");
    shape out{shape::int32_type, {static_cast<std::size_t>(v.cols)}};
    if(inputs[1] != out)
        MIGRAPHX_THROW("mi355::colsum: output buffer has the wrong shape");
    return out;
}

argument colsum::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const auto v = view_as_matrix(args[0].get_shape());
    status_check(mi355_colsum_i8(args[0].data(),
                                 v.rows,
                                 v.cols,
                                 v.ld,
                                 v.trans,
                                 reinterpret_cast<int32_t*>(args[1].data()),
                                 stream_of(ctx)),
                 name());
    return args[1];
}

shape rowsum::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    const auto v = view_as_matrix(inputs[0]);
    if(not v.ok or v.batch != 1 or inputs[0].type() != shape::int8_type)
        MIGRAPHX_THROW("mi355::rowsum: needs one int8 matrix");
    shape out{shape::int32_type, {static_cast<std::size_t>(v.rows)}};
    if(inputs[1] != out)
        MIGRAPHX_THROW("mi355::rowsum: output buffer has the wrong shape");
    return out;
}

argument rowsum::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const auto v = view_as_matrix(args[0].get_shape());
    status_check(mi355_rowsum_i8(args[0].data(),
                                 v.rows,
                                 v.cols,
                                 v.ld,
                                 v.trans,
                                 reinterpret_cast<int32_t*>(args[1].data()),
                                 stream_of(ctx)),
                 name());
    return args[1];
}

// ---- quant_dot_mx --------------------------------------------------------------------------

mi355_mx_dot_desc quant_dot_mx::describe(const std::vector<shape>& inputs) const
{
    if(inputs.size() != 6)
        MIGRAPHX_THROW("mi355::quant_dot_mx: expects a, b, scale_a, scale_b, workspace, out");
    const auto& a  = inputs[0];
    const auto& b  = inputs[1];
    const auto& sa = inputs[2];
    const auto& sb = inputs[3];
    const std::size_t nd = a.ndim();
    if(nd < 2 or b.ndim() != nd or not a.standard() or not b.standard())
        MIGRAPHX_THROW("mi355::quant_dot_mx: operands are standard tensors [.., M, K] and [.., N, K]");
    auto storage_ok = [](const shape& s, bool fp4) {
        return fp4 ? s.type() == shape::fp4x2_type : s.type() == shape::fp8e4m3fn_type;
    };
    if(not storage_ok(a, a_fp4) or not storage_ok(b, b_fp4))
        MIGRAPHX_THROW("mi355::quant_dot_mx: operand types are fp8e4m3fn or fp4x2");
    if(sa.type() != shape::float_type or sb.type() != shape::float_type)
        MIGRAPHX_THROW("mi355::quant_dot_mx: scales are float");
    mi355_mx_dot_desc d{};
    d.m     = static_cast<int64_t>(a.lens()[nd - 2]);
    d.n     = static_cast<int64_t>(b.lens()[nd - 2]);
    d.k     = static_cast<int64_t>(a.lens()[nd - 1]) * (a_fp4 ? 2 : 1);
    d.batch = 1;
    for(std::size_t i = 0; i + 2 < nd; i++)
    {
        if(a.lens()[i] != b.lens()[i])
            MIGRAPHX_THROW("mi355::quant_dot_mx: outer dimensions of A and B mismatch");
        d.batch *= static_cast<int64_t>(a.lens()[i]);
    }
    if(static_cast<int64_t>(b.lens()[nd - 1]) * (b_fp4 ? 2 : 1) != d.k)
        MIGRAPHX_THROW("mi355::quant_dot_mx: inner dimensions are not compatible");
    if(d.k % 32 != 0)
        MIGRAPHX_THROW("mi355::quant_dot_mx: K must be whole blocks of 32");
    d.lda      = static_cast<int64_t>(a.lens()[nd - 1]);
    d.ldb      = static_cast<int64_t>(b.lens()[nd - 1]);
    d.ldc      = d.n;
    d.stride_a = d.m * d.lda;
    d.stride_b = d.n * d.ldb;
    d.stride_c = d.m * d.n;
    d.a_type   = a_fp4 ? MI355_FP4X2 : MI355_FP8;
    d.b_type   = b_fp4 ? MI355_FP4X2 : MI355_FP8;
    // the one stride the batch dimensions of a view collapse into (0: no batch, or broadcast)
    auto batch_stride = [&](const shape& s) {
        int64_t r = 0;
        for(std::size_t i = 0; i + 2 < s.ndim(); i++)
        {
            if(s.lens()[i] > 1)
                r = static_cast<int64_t>(s.strides()[i]);
        }
        return r;
    };
    const auto nblk = d.k / 32;
    auto check_scale = [&](const shape& s, bool compact, int64_t rows, bool transposed) {
        if(s.ndim() != nd or not batch_collapses(s))
            MIGRAPHX_THROW("mi355::quant_dot_mx: scale has the wrong rank or batch layout");
        const auto r = static_cast<int64_t>(s.lens()[nd - 2]);
        const auto c = static_cast<int64_t>(s.lens()[nd - 1]);
        const bool ok = compact ? (s.standard() and r == rows and c == nblk)
                                : (transposed ? (r == d.k and c == rows) : (r == rows and c == d.k));
        if(not ok)
            MIGRAPHX_THROW("mi355::quant_dot_mx: scale has the wrong shape");
    };
    check_scale(sa, sa_compact, d.m, false);
    check_scale(sb, sb_compact, d.n, true);
    if(sa_compact)
    {
        d.sa_batch = d.m * nblk;
        d.sa_row   = nblk;
        d.sa_block = 1;
        d.sa_elem  = 0;
    }
    else
    {
        d.sa_batch = batch_stride(sa);
        d.sa_row   = static_cast<int64_t>(sa.strides()[nd - 2]);
        d.sa_elem  = static_cast<int64_t>(sa.strides()[nd - 1]);
        d.sa_block = 32 * d.sa_elem;
    }
    if(sb_compact)
    {
        d.sb_batch = d.n * nblk;
        d.sb_row   = nblk;
        d.sb_block = 1;
        d.sb_elem  = 0;
    }
    else
    {
        // scale_b has the operator's [.., K, N] shape
        d.sb_batch = batch_stride(sb);
        d.sb_elem  = static_cast<int64_t>(sb.strides()[nd - 2]);
        d.sb_row   = static_cast<int64_t>(sb.strides()[nd - 1]);
        d.sb_block = 32 * d.sb_elem;
    }
    return d;
}

shape quant_dot_mx::compute_shape(const std::vector<shape>& inputs) const
{
    const auto d = describe(inputs);
    auto lens    = inputs[0].lens();
    lens.back()  = static_cast<std::size_t>(d.n);
    shape out{shape::float_type, lens};
    if(inputs.back() != out)
        MIGRAPHX_THROW("mi355::quant_dot_mx: output buffer has the wrong shape");
    if(inputs[4].bytes() < mi355_quant_dot_mx_workspace_size(&d))
        MIGRAPHX_THROW("mi355::quant_dot_mx: workspace is too small");
    return out;
}

argument quant_dot_mx::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    std::vector<shape> shapes;
    for(const auto& a : args)
        shapes.push_back(a.get_shape());
    const auto d = describe(shapes);
    status_check(mi355_quant_dot_mx(&d,
                                    args[0].data(),
                                    args[1].data(),
                                    reinterpret_cast<float*>(args[5].data()),
                                    reinterpret_cast<const float*>(args[2].data()),
                                    reinterpret_cast<const float*>(args[3].data()),
                                    args[4].data(),
                                    args[4].get_shape().bytes(),
                                    stream_of(ctx)),
                 name());
    return args[5];
}

shape dot::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, scaled ? 4 : 3, name());
    auto s = op::dot{}.compute_shape({inputs[0], inputs[1]});
    to_mi355_type(s.type());
    if(scaled and (s.type() != shape::float_type or inputs[2].type() != shape::float_type or
                   inputs[2].elements() != 1))
        MIGRAPHX_THROW("mi355::dot: the scale is one float and needs a float dot");
    if(s.type() != shape::float_type and s.type() != shape::half_type and s.type() != shape::bf16_type)
        MIGRAPHX_THROW("mi355::dot: float, half or bf16 only");
    // any strides are fine inside a matrix; the batch dimensions must collapse into one stride, or
    // be two (each then keeps its own stride: the head split of an attention layer)
    for(int i = 0; i < 2; i++)
    {
        if(not batch_collapses(inputs[i]) and inputs[i].ndim() != 4)
            MIGRAPHX_THROW("mi355::dot: batch dimensions do not collapse into one stride");
    }
    // the result is dense, or (two batch axes, float) a view with rows of contiguous elements: the
    // [batch, heads, rows, width] result written into [batch, rows, heads, width] memory
    const shape& out = inputs.back();
    if(out == s)
        return s;
    if(out.type() != s.type() or out.lens() != s.lens() or s.ndim() != 4 or s.type() != shape::float_type or
       out.strides().back() != 1 or out.broadcasted())
        MIGRAPHX_THROW("mi355::dot: output buffer has the wrong shape");
    return out;
}

argument dot::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    const auto& sa       = args[0].get_shape();
    const auto& sb       = args[1].get_shape();
    const std::size_t nd = sa.ndim();
    const auto m         = static_cast<int64_t>(sa.lens()[nd - 2]);
    const auto k         = static_cast<int64_t>(sa.lens()[nd - 1]);
    const auto n         = static_cast<int64_t>(sb.lens()[nd - 1]);
    int64_t batch        = 1;
    for(std::size_t i = 0; i + 2 < nd; i++)
        batch *= static_cast<int64_t>(sa.lens()[i]);
    auto batch_stride = [&](const shape& s) {
        int64_t r = 0;
        for(std::size_t i = 0; i + 2 < nd; i++)
        {
            if(s.lens()[i] > 1)
                r = static_cast<int64_t>(s.strides()[i]);
        }
        return r;
    };
    const bool fast = fp32acc and out.type() == shape::float_type;
    if(nd == 4 and not out.standard())
    {
        status_check(mi355_dot_batch2_strided(args[0].data(),
                                              args[1].data(),
                                              args.back().data(),
                                              to_mi355_type(out.type()),
                                              m,
                                              n,
                                              k,
                                              static_cast<int64_t>(sa.strides()[2]),
                                              static_cast<int64_t>(sa.strides()[3]),
                                              static_cast<int64_t>(sb.strides()[2]),
                                              static_cast<int64_t>(sb.strides()[3]),
                                              static_cast<int64_t>(out.strides()[2]),
                                              static_cast<int64_t>(sa.lens()[0]),
                                              static_cast<int64_t>(sa.lens()[1]),
                                              static_cast<int64_t>(sa.strides()[0]),
                                              static_cast<int64_t>(sa.strides()[1]),
                                              static_cast<int64_t>(sb.strides()[0]),
                                              static_cast<int64_t>(sb.strides()[1]),
                                              static_cast<int64_t>(out.strides()[0]),
                                              static_cast<int64_t>(out.strides()[1]),
                                              scaled ? reinterpret_cast<const float*>(args[2].data()) : nullptr,
                                              fast ? 1 : 0,
                                              stream_of(ctx)),
                     name());
        return args.back();
    }
    if(nd == 4 and (not batch_collapses(sa) or not batch_collapses(sb)))
    {
        status_check(mi355_dot_batch2(args[0].data(),
                                      args[1].data(),
                                      args.back().data(),
                                      to_mi355_type(out.type()),
                                      m,
                                      n,
                                      k,
                                      static_cast<int64_t>(sa.strides()[2]),
                                      static_cast<int64_t>(sa.strides()[3]),
                                      static_cast<int64_t>(sb.strides()[2]),
                                      static_cast<int64_t>(sb.strides()[3]),
                                      static_cast<int64_t>(sa.lens()[0]),
                                      static_cast<int64_t>(sa.lens()[1]),
                                      static_cast<int64_t>(sa.strides()[0]),
                                      static_cast<int64_t>(sa.strides()[1]),
                                      static_cast<int64_t>(sb.strides()[0]),
                                      static_cast<int64_t>(sb.strides()[1]),
                                      scaled ? reinterpret_cast<const float*>(args[2].data()) : nullptr,
                                      fast ? 1 : 0,
                                      stream_of(ctx)),
                     name());
        return args.back();
    }
    status_check((fast ? mi355_dot_fp32acc : mi355_dot_scaled)(args[0].data(),
                           args[1].data(),
                           args.back().data(),
                           to_mi355_type(out.type()),
                           m,
                           n,
                           k,
                           static_cast<int64_t>(sa.strides()[nd - 2]),
                           static_cast<int64_t>(sa.strides()[nd - 1]),
                           static_cast<int64_t>(sb.strides()[nd - 2]),
                           static_cast<int64_t>(sb.strides()[nd - 1]),
                           n,
                           batch,
                           batch_stride(sa),
                           batch_stride(sb),
                           m * n,
                           scaled ? reinterpret_cast<const float*>(args[2].data()) : nullptr,
                           stream_of(ctx)),
                 name());
    return args.back();
}

shape w4a16_gemm::compute_shape(const std::vector<shape>& inputs) const
{
    const std::size_t expect = (zp_mode == MI355_W4_ZP_SCALAR ? 4 : 5) + (workspace ? 1 : 0);
    check_inputs(inputs, expect, name());
    if(workspace and inputs[inputs.size() - 2].type() != shape::uint8_type)
        MIGRAPHX_THROW("mi355::w4a16_gemm: the workspace must be a uint8 buffer");
    const auto& a = inputs[0];
    const auto& w = inputs[1];
    const auto& s = inputs[2];
    if(a.type() != shape::half_type or s.type() != shape::half_type or w.type() != shape::uint8_type)
        MIGRAPHX_THROW("mi355::w4a16_gemm: needs half activations and scales, uint8 packed weights");
    if(a.ndim() != 2 or w.ndim() != 2 or a.strides()[1] != 1 or not w.standard() or not s.standard())
        MIGRAPHX_THROW("mi355::w4a16_gemm: needs 2-D row-major operands");
    const auto k = a.lens()[1];
    const auto n = w.lens()[0];
    if(w.lens()[1] * 2 != k or group <= 0 or k % group != 0 or s.elements() != n * (k / group))
        MIGRAPHX_THROW("mi355::w4a16_gemm: operand dimensions do not fit");
    shape out{shape::half_type, {a.lens()[0], n}};
    if(inputs.back() != out)
        MIGRAPHX_THROW("mi355::w4a16_gemm: output buffer has the wrong shape");
    return out;
}

argument w4a16_gemm::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    const auto& a    = args[0].get_shape();
    const void* zp   = zp_mode == MI355_W4_ZP_SCALAR ? nullptr : args[3].data();
    const int64_t m  = static_cast<int64_t>(a.lens()[0]);
    const int64_t k  = static_cast<int64_t>(a.lens()[1]);
    const int64_t n  = static_cast<int64_t>(out.lens()[1]);
    const int64_t lda = m == 1 ? k : static_cast<int64_t>(a.strides()[0]);
    const auto& room = args[args.size() - 2];
    status_check(mi355_w4a16_gemm_ws(args[0].data(),
                                     lda,
                                     args[1].data(),
                                     args[2].data(),
                                     zp,
                                     static_cast<int32_t>(zp_mode),
                                     static_cast<int32_t>(zp_scalar),
                                     args.back().data(),
                                     n,
                                     m,
                                     n,
                                     k,
                                     group,
                                     workspace ? room.data() : nullptr,
                                     workspace ? room.get_shape().bytes() : 0,
                                     stream_of(ctx)),
                 name());
    return args.back();
}

shape w4a16_prepack::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 3, name());
    const auto& w = inputs[0];
    const auto& s = inputs[1];
    if(w.type() != shape::uint8_type or s.type() != shape::half_type or w.ndim() != 2 or not w.standard() or
       not s.standard())
        MIGRAPHX_THROW("mi355::w4a16_prepack: needs dense uint8 [N, K/2] weights and half scales");
    const auto n       = static_cast<int64_t>(w.lens()[0]);
    const auto k       = static_cast<int64_t>(w.lens()[1] * 2);
    const size_t bytes = mi355_w4a16_prepacked_size(n, k, 128);
    if(bytes == 0 or s.elements() != static_cast<std::size_t>(n * (k / 128)))
        MIGRAPHX_THROW("mi355::w4a16_prepack: the reordered form does not take this shape");
    shape out{shape::uint8_type, {bytes}};
    if(inputs.back() != out)
        MIGRAPHX_THROW("mi355::w4a16_prepack: output buffer has the wrong size");
    return out;
}

argument w4a16_prepack::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const auto& w = args[0].get_shape();
    status_check(mi355_w4a16_prepack(args[0].data(),
                                     args[1].data(),
                                     static_cast<int32_t>(zp_scalar),
                                     static_cast<int64_t>(w.lens()[0]),
                                     static_cast<int64_t>(w.lens()[1] * 2),
                                     128,
                                     args.back().data(),
                                     stream_of(ctx)),
                 name());
    return args.back();
}

shape w4a16_gemm_prepacked::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 3, name());
    const auto& a   = inputs[0];
    const auto& out = inputs.back();
    if(a.type() != shape::half_type or out.type() != shape::half_type or inputs[1].type() != shape::uint8_type)
        MIGRAPHX_THROW("mi355::w4a16_gemm_prepacked: needs half activations and a uint8 buffer of reordered weights");
    if(a.ndim() != 2 or out.ndim() != 2 or a.lens()[0] != out.lens()[0] or not out.standard() or
       (a.lens()[1] > 1 and a.strides()[1] != 1))
        MIGRAPHX_THROW("mi355::w4a16_gemm_prepacked: needs row-major activations and a dense result with the same rows");
    const auto max_rows =
        mi355_w4a16_prepacked_max_rows(static_cast<int64_t>(out.lens()[1]), static_cast<int64_t>(a.lens()[1]), 128);
    if(static_cast<int64_t>(a.lens()[0]) > max_rows)
        MIGRAPHX_THROW("mi355::w4a16_gemm_prepacked: takes at most " + std::to_string(max_rows) +
                       " rows of activations at this K");
    if(mi355_w4a16_prepacked_size(static_cast<int64_t>(out.lens()[1]), static_cast<int64_t>(a.lens()[1]), 128) !=
       inputs[1].bytes())
        MIGRAPHX_THROW("mi355::w4a16_gemm_prepacked: the reordered weights do not fit the operands");
    return out;
}

argument
w4a16_gemm_prepacked::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    const auto& a  = args[0].get_shape();
    const auto m   = static_cast<int64_t>(a.lens()[0]);
    const auto k   = static_cast<int64_t>(a.lens()[1]);
    const auto n   = static_cast<int64_t>(out.lens()[1]);
    const auto lda = m == 1 ? k : static_cast<int64_t>(a.strides()[0]);
    status_check(
        mi355_w4a16_gemm_prepacked(args[0].data(), lda, args[1].data(), args.back().data(), n, m, n, k, stream_of(ctx)),
        name());
    return args.back();
}

// ----------------------------------------------------------------- pointwise operators

shape quantizelinear::compute_shape(const std::vector<shape>& inputs) const
{
    if(inputs.size() != 3 and inputs.size() != 4)
        MIGRAPHX_THROW("mi355::quantizelinear: expected 3 or 4 arguments");
    check_standard(inputs[0], name());
    if(inputs[0].type() != inputs[1].type())
        MIGRAPHX_THROW("mi355::quantizelinear: Scales and input must be the same type");
    int64_t sr = 0;
    int64_t sc = 0;
    for(std::size_t i = 1; i + 1 < inputs.size(); i++)
    {
        if(inputs[i].lens() != inputs[0].lens() or not collapse_2d(inputs[i], sr, sc))
            MIGRAPHX_THROW("mi355::quantizelinear: parameter strides do not collapse to two");
    }
    if(inputs.size() == 4 and inputs[2].type() != out_type)
        MIGRAPHX_THROW("mi355::quantizelinear: zero point type differs from the output type");
    shape out{out_type, inputs[0].lens()};
    if(inputs.back() != out)
        MIGRAPHX_THROW("mi355::quantizelinear: output buffer has the wrong shape");
    return out;
}

argument
quantizelinear::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    int64_t rows = 0;
    int64_t cols = 0;
    rows_cols(out, rows, cols);
    int64_t s_sr = 0, s_sc = 0, z_sr = 0, z_sc = 0;
    collapse_2d(args[1].get_shape(), s_sr, s_sc);
    const void* zp = nullptr;
    if(args.size() == 4)
    {
        zp = args[2].data();
        collapse_2d(args[2].get_shape(), z_sr, z_sc);
    }
    status_check(mi355_quantizelinear(args[0].data(),
                                      to_mi355_type(args[0].get_shape().type()),
                                      args[1].data(),
                                      s_sr,
                                      s_sc,
                                      zp,
                                      z_sr,
                                      z_sc,
                                      args.back().data(),
                                      to_mi355_type(out.type()),
                                      rows,
                                      cols,
                                      stream_of(ctx)),
                 name());
    return args.back();
}

shape dequantizelinear::compute_shape(const std::vector<shape>& inputs) const
{
    if(inputs.size() != 3 and inputs.size() != 4)
        MIGRAPHX_THROW("mi355::dequantizelinear: expected 3 or 4 arguments");
    check_standard(inputs[0], name());
    int64_t sr = 0;
    int64_t sc = 0;
    for(std::size_t i = 1; i + 1 < inputs.size(); i++)
    {
        if(inputs[i].lens() != inputs[0].lens() or not collapse_2d(inputs[i], sr, sc))
            MIGRAPHX_THROW("mi355::dequantizelinear: parameter strides do not collapse to two");
    }
    if(inputs.size() == 4 and inputs[2].type() != inputs[0].type())
        MIGRAPHX_THROW("mi355::dequantizelinear: Zero point and input should be the same type.");
    shape out{inputs[1].type(), inputs[0].lens()};
    if(inputs.back() != out)
        MIGRAPHX_THROW("mi355::dequantizelinear: output buffer has the wrong shape");
    return out;
}

argument
dequantizelinear::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    int64_t rows = 0;
    int64_t cols = 0;
    rows_cols(out, rows, cols);
    int64_t s_sr = 0, s_sc = 0, z_sr = 0, z_sc = 0;
    collapse_2d(args[1].get_shape(), s_sr, s_sc);
    const void* zp = nullptr;
    if(args.size() == 4)
    {
        zp = args[2].data();
        collapse_2d(args[2].get_shape(), z_sr, z_sc);
    }
    status_check(mi355_dequantizelinear(args[0].data(),
                                        to_mi355_type(args[0].get_shape().type()),
                                        args[1].data(),
                                        to_mi355_type(args[1].get_shape().type()),
                                        s_sr,
                                        s_sc,
                                        zp,
                                        z_sr,
                                        z_sc,
                                        args.back().data(),
                                        rows,
                                        cols,
                                        stream_of(ctx)),
                 name());
    return args.back();
}

shape unpack_int4::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    op::unpack_int4 ref;
    ref.axis = axis;
    auto out = ref.compute_shape({inputs[0]});
    if(inputs[1] != out)
        MIGRAPHX_THROW("mi355::unpack_int4: output buffer has the wrong shape");
    return out;
}

// lengths and element strides of a view as the C ABI takes them
static void lens_strides(const shape& s, std::vector<int64_t>& lens, std::vector<int64_t>& strides)
{
    lens.assign(s.lens().begin(), s.lens().end());
    strides.assign(s.strides().begin(), s.strides().end());
}

argument unpack_int4::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const auto& in = args[0].get_shape();
    const auto nd  = static_cast<int64_t>(in.ndim());
    if(in.standard() and (axis == -1 or axis == nd - 1))
    {
        int64_t rows = 0;
        int64_t cols = 0;
        rows_cols(in, rows, cols);
        status_check(mi355_unpack_int4(args[0].data(), args[1].data(), in.type() == shape::int8_type, rows, cols,
                                       stream_of(ctx)),
                     name());
        return args[1];
    }
    if(nd > MI355_MAX_DIMS)
        MIGRAPHX_THROW("mi355::unpack_int4: more than 8 dimensions");
    std::vector<int64_t> lens, strides;
    lens_strides(in, lens, strides);
    status_check(mi355_unpack_int4_nd(args[0].data(), args[1].data(), in.type() == shape::int8_type,
                                      static_cast<int32_t>(nd), lens.data(), strides.data(),
                                      static_cast<int32_t>(axis), stream_of(ctx)),
                 name());
    return args[1];
}

shape unpack_fp4::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    check_standard(inputs[0], name());
    auto out = op::unpack_fp4{}.compute_shape({inputs[0]});
    if(inputs[1] != out)
        MIGRAPHX_THROW("mi355::unpack_fp4: output buffer has the wrong shape");
    return out;
}

argument unpack_fp4::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    int64_t rows = 0;
    int64_t cols = 0;
    rows_cols(args[0].get_shape(), rows, cols);
    status_check(mi355_unpack_fp4(args[0].data(), args[1].data(), rows, cols, stream_of(ctx)), name());
    return args[1];
}

shape pack_fp4::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    check_standard(inputs[0], name());
    if(inputs[0].type() != shape::float_type)
        MIGRAPHX_THROW("mi355::pack_fp4: the kernel takes float input");
    auto out = op::pack_fp4{}.compute_shape({inputs[0]});
    if(inputs[1] != out)
        MIGRAPHX_THROW("mi355::pack_fp4: output buffer has the wrong shape");
    return out;
}

argument pack_fp4::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    int64_t rows = 0;
    int64_t cols = 0;
    rows_cols(args[0].get_shape(), rows, cols);
    status_check(mi355_pack_fp4(reinterpret_cast<const float*>(args[0].data()), args[1].data(), rows, cols,
                                stream_of(ctx)),
                 name());
    return args[1];
}

shape pack_int4::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    op::pack_int4 ref;
    ref.axis = axis;
    auto out = ref.compute_shape({inputs[0]});
    if(inputs[1] != out)
        MIGRAPHX_THROW("mi355::pack_int4: output buffer has the wrong shape");
    return out;
}

argument pack_int4::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const auto& in = args[0].get_shape();
    const auto nd  = static_cast<int64_t>(in.ndim());
    if(in.standard() and (axis == -1 or axis == nd - 1))
    {
        int64_t rows = 0;
        int64_t cols = 0;
        rows_cols(in, rows, cols);
        status_check(mi355_pack_int4(args[0].data(), args[1].data(), in.type() == shape::int8_type, rows, cols,
                                     stream_of(ctx)),
                     name());
        return args[1];
    }
    if(nd > MI355_MAX_DIMS)
        MIGRAPHX_THROW("mi355::pack_int4: more than 8 dimensions");
    std::vector<int64_t> lens, strides;
    lens_strides(in, lens, strides);
    status_check(mi355_pack_int4_nd(args[0].data(), args[1].data(), in.type() == shape::int8_type,
                                    static_cast<int32_t>(nd), lens.data(), strides.data(),
                                    static_cast<int32_t>(axis), stream_of(ctx)),
                 name());
    return args[1];
}

shape convert::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    check_standard(inputs[0], name());
    shape out{target_type, inputs[0].lens()};
    if(inputs[1] != out)
        MIGRAPHX_THROW("mi355::convert: output buffer has the wrong shape");
    return out;
}

argument convert::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    status_check(mi355_convert(args[0].data(),
                               to_mi355_type(args[0].get_shape().type()),
                               args[1].data(),
                               to_mi355_type(out.type()),
                               static_cast<int64_t>(out.elements()),
                               stream_of(ctx)),
                 name());
    return args[1];
}

shape contiguous::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    if(inputs[0].ndim() > MI355_MAX_DIMS)
        MIGRAPHX_THROW("mi355::contiguous: too many dimensions");
    shape out{inputs[0].type(), inputs[0].lens()};
    if(inputs[1] != out)
        MIGRAPHX_THROW("mi355::contiguous: output buffer has the wrong shape");
    return out;
}

argument contiguous::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const auto& s = args[0].get_shape();
    std::vector<int64_t> lens(s.lens().begin(), s.lens().end());
    std::vector<int64_t> strides(s.strides().begin(), s.strides().end());
    status_check(mi355_contiguous(args[0].data(),
                                  args[1].data(),
                                  static_cast<int32_t>(s.type_size()),
                                  static_cast<int32_t>(s.ndim()),
                                  lens.data(),
                                  strides.data(),
                                  stream_of(ctx)),
                 name());
    return args[1];
}

// ----------------------------------------------------------------- float operators

shape binary::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 3, name());
    const auto t = inputs[0].type();
    const bool narrow_int = t == shape::int8_type or t == shape::uint8_type;
    const bool narrow_flt = t == shape::half_type or t == shape::bf16_type;
    if(t != inputs[1].type() or
       (t != shape::float_type and t != shape::int32_type and not narrow_int and not narrow_flt))
        MIGRAPHX_THROW("mi355::binary: float, half, bf16, int32, int8 or uint8 tensors of one type only, got " +
                       inputs[0].type_string() + " and " + inputs[1].type_string());
    if((t == shape::int32_type or narrow_int) and op == MI355_BIN_DIV)
        MIGRAPHX_THROW("mi355::binary: integer division has no kernel");
    if(t != shape::float_type and (op == MI355_BIN_MAX or op == MI355_BIN_MIN))
        MIGRAPHX_THROW("mi355::binary: max and min have a float kernel only");
    if(inputs[0].lens() != inputs[1].lens())
        MIGRAPHX_THROW("mi355::binary: Dimensions do not match");
    if(inputs[0].ndim() > MI355_MAX_DIMS)
        MIGRAPHX_THROW("mi355::binary: too many dimensions");
    shape out{t, inputs[0].lens()};
    if(inputs[2] != out)
        MIGRAPHX_THROW("mi355::binary: output buffer has the wrong shape");
    return out;
}

argument binary::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    std::vector<int64_t> lens(out.lens().begin(), out.lens().end());
    auto strides_of = [&](const shape& s) {
        std::vector<int64_t> r(s.strides().begin(), s.strides().end());
        for(std::size_t i = 0; i < r.size(); i++)
        {
            if(s.lens()[i] == 1)
                r[i] = 0;
        }
        return r;
    };
    const auto sa = strides_of(args[0].get_shape());
    const auto sb = strides_of(args[1].get_shape());
    if(out.type() != shape::int32_type and out.type() != shape::float_type)
    {
        status_check(mi355_binary_typed(static_cast<int32_t>(op),
                                        to_mi355_type(out.type()),
                                        args[0].data(),
                                        sa.data(),
                                        args[1].data(),
                                        sb.data(),
                                        args[2].data(),
                                        static_cast<int32_t>(lens.size()),
                                        lens.data(),
                                        stream_of(ctx)),
                     name());
        return args[2];
    }
    if(out.type() == shape::int32_type)
    {
        status_check(mi355_binary_i32(static_cast<int32_t>(op),
                                      reinterpret_cast<const int32_t*>(args[0].data()),
                                      sa.data(),
                                      reinterpret_cast<const int32_t*>(args[1].data()),
                                      sb.data(),
                                      reinterpret_cast<int32_t*>(args[2].data()),
                                      static_cast<int32_t>(lens.size()),
                                      lens.data(),
                                      stream_of(ctx)),
                     name());
        return args[2];
    }
    status_check(mi355_binary_f32(static_cast<int32_t>(op),
                                  reinterpret_cast<const float*>(args[0].data()),
                                  sa.data(),
                                  reinterpret_cast<const float*>(args[1].data()),
                                  sb.data(),
                                  reinterpret_cast<float*>(args[2].data()),
                                  static_cast<int32_t>(lens.size()),
                                  lens.data(),
                                  stream_of(ctx)),
                 name());
    return args[2];
}

shape unary::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    check_standard(inputs[0], name());
    if(inputs[0].type() != shape::float_type)
        MIGRAPHX_THROW("mi355::unary: float tensors only");
    if(inputs[1] != inputs[0])
        MIGRAPHX_THROW("mi355::unary: output buffer has the wrong shape");
    return inputs[0];
}

argument unary::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    status_check(mi355_unary_f32(static_cast<int32_t>(op),
                                 reinterpret_cast<const float*>(args[0].data()),
                                 reinterpret_cast<float*>(args[1].data()),
                                 static_cast<int64_t>(out.elements()),
                                 stream_of(ctx)),
                 name());
    return args[1];
}

namespace {
// the host arrays the chain entry points take: steps, and a pointer, a row stride and a column
// stride for each of the first n arguments
struct chain_call
{
    std::vector<mi355_chain_step> st;
    std::vector<const float*> ptrs;
    std::vector<int64_t> sr;
    std::vector<int32_t> sc;
    chain_call(const std::vector<int64_t>& steps, const std::vector<argument>& args, std::size_t n)
        : st(steps.size() / 4), ptrs(n), sr(n), sc(n)
    {
        for(std::size_t i = 0; i < st.size(); i++)
        {
            st[i].kind     = static_cast<int32_t>(steps[4 * i]);
            st[i].op       = static_cast<int32_t>(steps[4 * i + 1]);
            st[i].src      = static_cast<int32_t>(steps[4 * i + 2]);
            st[i].reversed = static_cast<int32_t>(steps[4 * i + 3]);
        }
        for(std::size_t i = 0; i < n; i++)
        {
            int64_t r = 0;
            int64_t c = 0;
            collapse_2d(args[i].get_shape(), r, c);
            ptrs[i] = reinterpret_cast<const float*>(args[i].data());
            sr[i]   = r;
            sc[i]   = static_cast<int32_t>(c);
        }
    }
};
} // namespace

shape chain::compute_shape(const std::vector<shape>& inputs) const
{
    if(inputs.size() < 2 or inputs.size() > MI355_CHAIN_MAX_INPUTS + 1)
        MIGRAPHX_THROW("mi355::chain: between 1 and " + std::to_string(MI355_CHAIN_MAX_INPUTS) +
                       " inputs and the output buffer expected");
    if(steps.empty() or steps.size() % 4 != 0 or steps.size() / 4 > MI355_CHAIN_MAX_STEPS)
        MIGRAPHX_THROW("mi355::chain: malformed step list");
    const shape& out = inputs.back();
    if(out.type() != shape::float_type or not out.standard())
        MIGRAPHX_THROW("mi355::chain: the output buffer must be a dense float tensor");
    for(std::size_t i = 0; i + 1 < inputs.size(); i++)
    {
        int64_t sr = 0;
        int64_t sc = 0;
        if(inputs[i].type() != shape::float_type)
            MIGRAPHX_THROW("mi355::chain: float tensors only, got " + inputs[i].type_string());
        if(inputs[i].lens() != out.lens())
            MIGRAPHX_THROW("mi355::chain: Dimensions do not match");
        if(not collapse_2d(inputs[i], sr, sc) or (sc != 0 and sc != 1))
            MIGRAPHX_THROW("mi355::chain: input strides do not collapse to rows and columns");
    }
    return out;
}

argument chain::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    const std::size_t n = args.size() - 1;
    chain_call c(steps, args, n);
    int64_t rows = 0;
    int64_t cols = 0;
    rows_cols(out, rows, cols);
    status_check(mi355_chain_f32(c.st.data(),
                                 static_cast<int32_t>(c.st.size()),
                                 c.ptrs.data(),
                                 c.sr.data(),
                                 c.sc.data(),
                                 static_cast<int32_t>(n),
                                 reinterpret_cast<float*>(args[n].data()),
                                 rows,
                                 cols,
                                 stream_of(ctx)),
                 name());
    return args[n];
}

shape chain_rows::compute_shape(const std::vector<shape>& inputs) const
{
    if(inputs.size() < 2 or inputs.size() > MI355_CHAIN_MAX_INPUTS + 1)
        MIGRAPHX_THROW("mi355::chain_rows: between 1 and " + std::to_string(MI355_CHAIN_MAX_INPUTS) +
                       " inputs and the output buffer expected");
    if(steps.empty() or steps.size() % 4 != 0 or steps.size() / 4 > MI355_CHAIN_MAX_STEPS)
        MIGRAPHX_THROW("mi355::chain_rows: malformed step list");
    const shape& out = inputs.back();
    if(out.type() != shape::float_type or not out.standard() or out.ndim() == 0)
        MIGRAPHX_THROW("mi355::chain_rows: the output buffer must be a dense float tensor");
    if(out.lens().back() > MI355_CHAIN_ROWS_MAX_COLS)
        MIGRAPHX_THROW("mi355::chain_rows: rows of at most " + std::to_string(MI355_CHAIN_ROWS_MAX_COLS) + " elements");
    // an input has the result's dimensions, or one value per row (last dimension 1)
    auto per_row = out.lens();
    per_row.back() = 1;
    for(std::size_t i = 0; i + 1 < inputs.size(); i++)
    {
        int64_t sr = 0;
        int64_t sc = 0;
        if(inputs[i].type() != shape::float_type)
            MIGRAPHX_THROW("mi355::chain_rows: float tensors only, got " + inputs[i].type_string());
        if(inputs[i].lens() != out.lens() and inputs[i].lens() != per_row)
            MIGRAPHX_THROW("mi355::chain_rows: Dimensions do not match");
        if(not collapse_2d(inputs[i], sr, sc) or (sc != 0 and sc != 1))
            MIGRAPHX_THROW("mi355::chain_rows: input strides do not collapse to rows and columns");
    }
    return out;
}

argument chain_rows::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    const std::size_t n = args.size() - 1;
    chain_call c(steps, args, n);
    int64_t rows = 0;
    int64_t cols = 0;
    rows_cols(out, rows, cols);
    status_check(mi355_chain_rows_f32(c.st.data(),
                                      static_cast<int32_t>(c.st.size()),
                                      c.ptrs.data(),
                                      c.sr.data(),
                                      c.sc.data(),
                                      static_cast<int32_t>(n),
                                      reinterpret_cast<float*>(args[n].data()),
                                      rows,
                                      cols,
                                      stream_of(ctx)),
                 name());
    return args[n];
}

shape chain_q8::compute_shape(const std::vector<shape>& inputs) const
{
    const std::size_t extra = has_zero_point ? 3 : 2; // scale, [zero point], out
    if(inputs.size() < extra + 1 or inputs.size() > MI355_CHAIN_MAX_INPUTS + extra)
        MIGRAPHX_THROW("mi355::chain_q8: between 1 and " + std::to_string(MI355_CHAIN_MAX_INPUTS) +
                       " inputs, the scale, the zero point if any and the output buffer expected");
    if(steps.empty() or steps.size() % 4 != 0 or steps.size() / 4 > MI355_CHAIN_MAX_STEPS)
        MIGRAPHX_THROW("mi355::chain_q8: malformed step list");
    const shape& out = inputs.back();
    if(out.type() != shape::int8_type or not out.standard())
        MIGRAPHX_THROW("mi355::chain_q8: the output buffer must be a dense int8 tensor");
    const std::size_t n = inputs.size() - extra;
    for(std::size_t i = 0; i < n; i++)
    {
        int64_t sr = 0;
        int64_t sc = 0;
        if(inputs[i].type() != shape::float_type)
            MIGRAPHX_THROW("mi355::chain_q8: float tensors only, got " + inputs[i].type_string());
        if(inputs[i].lens() != out.lens())
            MIGRAPHX_THROW("mi355::chain_q8: Dimensions do not match");
        if(not collapse_2d(inputs[i], sr, sc) or (sc != 0 and sc != 1))
            MIGRAPHX_THROW("mi355::chain_q8: input strides do not collapse to rows and columns");
    }
    if(inputs[n].type() != shape::float_type)
        MIGRAPHX_THROW("mi355::chain_q8: the scale is a float");
    if(has_zero_point and inputs[n + 1].type() != shape::int8_type)
        MIGRAPHX_THROW("mi355::chain_q8: the zero point is an int8");
    return out;
}

argument chain_q8::compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const
{
    const std::size_t extra = has_zero_point ? 3 : 2;
    const std::size_t n     = args.size() - extra;
    chain_call c(steps, args, n);
    int64_t rows = 0;
    int64_t cols = 0;
    rows_cols(out, rows, cols);
    status_check(mi355_chain_f32_q8(c.st.data(),
                                    static_cast<int32_t>(c.st.size()),
                                    c.ptrs.data(),
                                    c.sr.data(),
                                    c.sc.data(),
                                    static_cast<int32_t>(n),
                                    reinterpret_cast<const float*>(args[n].data()),
                                    has_zero_point ? reinterpret_cast<const int8_t*>(args[n + 1].data()) : nullptr,
                                    reinterpret_cast<int8_t*>(args.back().data()),
                                    rows,
                                    cols,
                                    stream_of(ctx)),
                 name());
    return args.back();
}

shape reduce_mean::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    check_standard(inputs[0], name());
    if(inputs[0].type() != shape::float_type)
        MIGRAPHX_THROW("mi355::reduce_mean: float tensors only");
    auto lens   = inputs[0].lens();
    lens.back() = 1;
    shape out{shape::float_type, lens};
    if(inputs[1] != out)
        MIGRAPHX_THROW("mi355::reduce_mean: output buffer has the wrong shape");
    return out;
}

argument reduce_mean::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    int64_t rows = 0;
    int64_t cols = 0;
    rows_cols(args[0].get_shape(), rows, cols);
    status_check(mi355_reduce_mean_f32(reinterpret_cast<const float*>(args[0].data()),
                                       reinterpret_cast<float*>(args[1].data()),
                                       rows,
                                       cols,
                                       stream_of(ctx)),
                 name());
    return args[1];
}

shape reduce_all::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    check_standard(inputs[0], name());
    if(inputs[0].type() != shape::float_type or inputs[1].type() != shape::float_type)
        MIGRAPHX_THROW("mi355::reduce_all: float tensors only");
    if(inputs[0].elements() == 0 or inputs[1].elements() != 1 or (op != 0 and op != 1))
        MIGRAPHX_THROW("mi355::reduce_all: reduces a tensor that is not empty to one element (op 0: max, 1: min)");
    return inputs[1];
}

argument reduce_all::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    status_check(mi355_reduce_all_f32(static_cast<int32_t>(op),
                                      reinterpret_cast<const float*>(args[0].data()),
                                      reinterpret_cast<float*>(args[1].data()),
                                      static_cast<int64_t>(args[0].get_shape().elements()),
                                      stream_of(ctx)),
                 name());
    return args[1];
}

shape softmax::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 2, name());
    check_standard(inputs[0], name());
    if(inputs[0].type() != shape::float_type)
        MIGRAPHX_THROW("mi355::softmax: float tensors only");
    if(inputs[1] != inputs[0])
        MIGRAPHX_THROW("mi355::softmax: output buffer has the wrong shape");
    return inputs[0];
}

argument softmax::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    int64_t rows = 0;
    int64_t cols = 0;
    rows_cols(args[0].get_shape(), rows, cols);
    status_check(mi355_softmax_f32(reinterpret_cast<const float*>(args[0].data()),
                                   reinterpret_cast<float*>(args[1].data()),
                                   rows,
                                   cols,
                                   stream_of(ctx)),
                 name());
    return args[1];
}

shape gather::compute_shape(const std::vector<shape>& inputs) const
{
    check_inputs(inputs, 3, name());
    check_standard(inputs[0], name());
    check_standard(inputs[1], name());
    if(inputs[1].type() != shape::int32_type and inputs[1].type() != shape::int64_type)
        MIGRAPHX_THROW("mi355::gather: indices must be int32 or int64");
    auto out = op::gather{}.compute_shape({inputs[0], inputs[1]});
    if((inputs[0].bytes() / inputs[0].lens()[0]) % 4 != 0)
        MIGRAPHX_THROW("mi355::gather: rows must be a multiple of 4 bytes");
    if(inputs[2] != out)
        MIGRAPHX_THROW("mi355::gather: output buffer has the wrong shape");
    return out;
}

argument gather::compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const
{
    const auto& t = args[0].get_shape();
    status_check(mi355_gather_rows(args[0].data(),
                                   args[1].data(),
                                   args[1].get_shape().type() == shape::int64_type,
                                   args[2].data(),
                                   static_cast<int64_t>(args[1].get_shape().elements()),
                                   static_cast<int64_t>(t.lens()[0]),
                                   static_cast<int64_t>(t.bytes() / t.lens()[0]),
                                   stream_of(ctx)),
                 name());
    return args[2];
}

// ----------------------------------------------------------------- target

std::vector<pass> target::get_passes(migraphx::context& gctx, const compile_options& options) const
{
    auto& ctx = any_cast<context>(gctx);
    // gfx950 has the block-scaled matrix instructions, so the MX rewrite is on, as the reference's
    // gpu target switches it (src/targets/gpu/target.cpp:129)
    simplify_qdq sq;
    sq.use_mx_quant = true;
    lowering low{&ctx, options.offload_copy};
    // the reference's switch for its pointwise fusion (src/fuse_pointwise.cpp:39,369)
    if(const char* off = std::getenv("MIGRAPHX_DISABLE_POINTWISE_FUSION"))
        low.fuse_pointwise = std::string(off).empty() or std::string(off) == "0";
    // MIGRAPHX_MI355_DISABLE_MEMORY_COLORING: every intermediate buffer keeps an allocation of its own
    if(const char* off = std::getenv("MIGRAPHX_MI355_DISABLE_MEMORY_COLORING"))
    {
        if(not std::string(off).empty() and std::string(off) != "0")
            return {sq, dead_code_elimination{}, low, dead_code_elimination{}};
    }
    return {sq, dead_code_elimination{}, low, dead_code_elimination{}, memory_coloring{}};
}

} // namespace mi355

MIGRAPHX_REGISTER_OP(mi355::allocate);
MIGRAPHX_REGISTER_OP(mi355::chain_q8);
MIGRAPHX_REGISTER_OP(mi355::chain_rows);
MIGRAPHX_REGISTER_OP(mi355::arena);
MIGRAPHX_REGISTER_OP(mi355::load);
MIGRAPHX_REGISTER_OP(mi355::device_literal);
MIGRAPHX_REGISTER_OP(mi355::copy_to_device);
MIGRAPHX_REGISTER_OP(mi355::copy_from_device);
MIGRAPHX_REGISTER_OP(mi355::quant_dot);
MIGRAPHX_REGISTER_OP(mi355::quant_convolution);
MIGRAPHX_REGISTER_OP(mi355::colsum);
MIGRAPHX_REGISTER_OP(mi355::rowsum);
MIGRAPHX_REGISTER_OP(mi355::dot);
MIGRAPHX_REGISTER_OP(mi355::quant_dot_mx);
MIGRAPHX_REGISTER_OP(mi355::w4a16_gemm);
MIGRAPHX_REGISTER_OP(mi355::convolution);
MIGRAPHX_REGISTER_OP(mi355::w4a16_prepack);
MIGRAPHX_REGISTER_OP(mi355::quant_dot_prepack);
MIGRAPHX_REGISTER_OP(mi355::quant_dot_prepacked);
MIGRAPHX_REGISTER_OP(mi355::w4a16_gemm_prepacked);
MIGRAPHX_REGISTER_OP(mi355::quantizelinear);
MIGRAPHX_REGISTER_OP(mi355::dequantizelinear);
MIGRAPHX_REGISTER_OP(mi355::chain);
MIGRAPHX_REGISTER_OP(mi355::unpack_int4);
MIGRAPHX_REGISTER_OP(mi355::unpack_fp4);
MIGRAPHX_REGISTER_OP(mi355::pack_fp4);
MIGRAPHX_REGISTER_OP(mi355::pack_int4);
MIGRAPHX_REGISTER_OP(mi355::convert);
MIGRAPHX_REGISTER_OP(mi355::contiguous);
MIGRAPHX_REGISTER_OP(mi355::binary);
MIGRAPHX_REGISTER_OP(mi355::unary);
MIGRAPHX_REGISTER_OP(mi355::reduce_mean);
MIGRAPHX_REGISTER_OP(mi355::reduce_all);
MIGRAPHX_REGISTER_OP(mi355::softmax);
MIGRAPHX_REGISTER_OP(mi355::gather);
MIGRAPHX_REGISTER_TARGET(mi355::target);

} // namespace migraphx
