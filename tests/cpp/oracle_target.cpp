#include "oracle_target.hpp"
#include <migraphx/ops.hpp>
#include <migraphx/passes.hpp>
#include <migraphx/register_target.hpp>
#include <cstdint>
#include <cmath>
#include <cstring>
#include <limits>

extern "C" {
// oracle/ref_oracle.c
void orc_gemm(void* c, int c_type, const void* a, const void* b, int ab_type, int64_t m, int64_t n,
              int64_t k, int64_t a_sm, int64_t a_sk, int64_t b_sk, int64_t b_sn, int64_t batch,
              int64_t a_sb, int64_t b_sb);
void orc_convolution3d(void* out, int out_type, const void* x, const void* w, int x_type, int64_t n,
                       int64_t c, const int64_t* in_lens, int64_t o, const int64_t* win_lens,
                       const int64_t* pad, const int64_t* stride, const int64_t* dil, int64_t group,
                       const int64_t* out_lens);
void orc_quantizelinear(void* out, int out_type, const void* x, int x_type, const void* scale,
                        int64_t s_sr, int64_t s_sc, const void* zp, int64_t z_sr, int64_t z_sc,
                        int64_t rows, int64_t cols);
void orc_dequantizelinear(void* out, const void* x, int x_type, const void* scale, int s_type,
                          int64_t s_sr, int64_t s_sc, const void* zp, int64_t z_sr, int64_t z_sc,
                          int64_t rows, int64_t cols);
void orc_unpack_int4(uint8_t* out, const uint8_t* in, int is_signed, int64_t outer, int64_t axis_len,
                     int64_t inner);
void orc_pack_int4(uint8_t* out, const uint8_t* in, int is_signed, int64_t outer, int64_t axis_len,
                   int64_t inner);
void orc_convert(void* out, int out_type, const void* x, int x_type, size_t n);
void orc_unpack_fp4(uint8_t* out, const uint8_t* in, int64_t outer, int64_t axis_len, int64_t inner);
void orc_pack_fp4(uint8_t* out, const float* in, int64_t outer, int64_t axis_len, int64_t inner);
void orc_binary_f32(int op, float* out, const float* a, const float* b, size_t n);
void orc_unary_f32(int op, float* out, const float* x, size_t n);
void orc_reduce_mean_f32(float* out, const float* x, int64_t outer, int64_t axis_len, int64_t inner);
void orc_softmax_f32(float* out, const float* x, int64_t outer, int64_t axis_len, int64_t inner);
void orc_gather(void* out, const void* data, const int64_t* idx, int64_t n_idx, int64_t outer,
                int64_t axis_len, int64_t inner, int64_t elem_size);
}

namespace oracle {

using migraphx::argument;
using migraphx::shape;

namespace {

enum
{
    ORC_I8,
    ORC_U8,
    ORC_I32,
    ORC_F32,
    ORC_F16,
    ORC_BF16,
    ORC_FP8,
    ORC_F64,
    ORC_BF8
};

int orc_type(shape::type_t t)
{
    switch(t)
    {
    case shape::int8_type: return ORC_I8;
    case shape::uint8_type: return ORC_U8;
    case shape::int32_type: return ORC_I32;
    case shape::float_type: return ORC_F32;
    case shape::half_type: return ORC_F16;
    case shape::bf16_type: return ORC_BF16;
    case shape::fp8e4m3fn_type: return ORC_FP8;
    case shape::fp8e5m2_type: return ORC_BF8;
    case shape::double_type: return ORC_F64;
    default: MIGRAPHX_THROW("oracle: unsupported type " + shape::type_name(t));
    }
}

argument dense(const argument& a)
{
    if(a.get_shape().standard())
        return a;
    return migraphx::op::contiguous{}.compute(
        shape{a.get_shape().type(), a.get_shape().lens()}, {a});
}

void rows_cols(const shape& s, int64_t& rows, int64_t& cols)
{
    cols = static_cast<int64_t>(s.lens().back());
    rows = cols == 0 ? 0 : static_cast<int64_t>(s.elements()) / cols;
}

// Evaluates the wrapped reference operator on host memory.
struct cpu_op
{
    migraphx::operation op;
    std::string name() const { return "oracle::" + op.name(); }
    // saved with the wrapped operator's own fields
    migraphx::value to_value() const { return op.to_value(); }
    void from_value(const migraphx::value& v) { op.from_value(v); }
    shape compute_shape(const std::vector<shape>& inputs) const
    {
        auto s = op.compute_shape(inputs);
        return shape{s.type(), s.lens()};
    }
    argument compute(migraphx::context&, const shape& out, const std::vector<argument>& args) const
    {
        const auto n = op.name();
        argument r{out};
        if(n == "quant_dot" or n == "dot")
        {
            // batches are gathered to dense tensors; inside a matrix the strides are used as
            // they are, so that transposed views reach the GEMM untouched
            argument a = args[0];
            argument b = args[1];
            if(args.size() == 4)
            {
                // four-input quant_dot (ref/lowering.cpp:221-242): float(x) * float(scale), element
                // by element, then the float GEMM
                auto scaled = [&](const argument& x, const argument& sc) {
                    const argument xd = dense(x);
                    const argument sd = dense(sc);
                    const shape fs{shape::float_type, xd.get_shape().lens()};
                    argument xf{fs};
                    argument sf{fs};
                    argument prod{fs};
                    orc_convert(xf.data(), orc_type(shape::float_type), xd.data(),
                                orc_type(xd.get_shape().type()), fs.elements());
                    orc_convert(sf.data(), orc_type(shape::float_type), sd.data(),
                                orc_type(sd.get_shape().type()), fs.elements());
                    orc_binary_f32(2, reinterpret_cast<float*>(prod.data()),
                                   reinterpret_cast<const float*>(xf.data()),
                                   reinterpret_cast<const float*>(sf.data()), fs.elements());
                    return prod;
                };
                a = scaled(args[0], args[2]);
                b = scaled(args[1], args[3]);
            }
            if(a.get_shape().ndim() > 2)
            {
                a = dense(a);
                b = dense(b);
            }
            const auto& sa       = a.get_shape();
            const auto& sb       = b.get_shape();
            const std::size_t nd = sa.ndim();
            const int64_t m      = sa.lens()[nd - 2];
            const int64_t k      = sa.lens()[nd - 1];
            const int64_t nn     = sb.lens()[nd - 1];
            const int64_t batch  = m * k == 0 ? 0 : sa.elements() / (m * k);
            orc_gemm(r.data(), orc_type(out.type()), a.data(), b.data(), orc_type(sa.type()), m, nn, k,
                     sa.strides()[nd - 2], sa.strides()[nd - 1], sb.strides()[nd - 2],
                     sb.strides()[nd - 1], batch, nd > 2 ? m * k : 0, nd > 2 ? k * nn : 0);
        }
        else if(n == "convolution" or n == "quant_convolution")
        {
            // one to three spatial dimensions; missing leading ones have length one
            const auto v        = op.to_value();
            const auto padding  = v.at("padding").to_vector<int64_t>();
            const auto stride   = v.at("stride").to_vector<int64_t>();
            const auto dilation = v.at("dilation").to_vector<int64_t>();
            const std::size_t kd = stride.size();
            if(args.size() != 2 or kd < 1 or kd > 3)
                MIGRAPHX_THROW("oracle: convolution with " + std::to_string(kd) + " spatial dimensions");
            argument x = dense(args[0]);
            argument w = dense(args[1]);
            const auto& xl = x.get_shape().lens();
            const auto& wl = w.get_shape().lens();
            const std::size_t lead = 3 - kd;
            int64_t in[3] = {1, 1, 1}, win[3] = {1, 1, 1}, pad[3] = {0, 0, 0}, st[3] = {1, 1, 1},
                    dil[3] = {1, 1, 1}, ol[3] = {1, 1, 1};
            for(std::size_t i = 0; i < kd; i++)
            {
                in[lead + i]  = xl[2 + i];
                win[lead + i] = wl[2 + i];
                pad[lead + i] = padding[i]; // the low side; the high side only enters the output size
                st[lead + i]  = stride[i];
                dil[lead + i] = dilation[i];
                ol[lead + i]  = out.lens()[2 + i];
            }
            orc_convolution3d(r.data(), orc_type(out.type()), x.data(), w.data(), orc_type(x.get_shape().type()),
                              xl[0], xl[1], in, wl[0], win, pad, st, dil, v.at("group").to<int64_t>(), ol);
        }
        else if(n == "quantizelinear" or n == "dequantizelinear")
        {
            int64_t rows = 0;
            int64_t cols = 0;
            rows_cols(out, rows, cols);
            argument x  = dense(args[0]);
            argument s  = dense(args[1]);
            argument zp = args.size() > 2 ? dense(args[2]) : argument{};
            if(n == "quantizelinear")
                orc_quantizelinear(r.data(), orc_type(out.type()), x.data(),
                                   orc_type(x.get_shape().type()), s.data(), cols, 1,
                                   zp.empty() ? nullptr : zp.data(), cols, 1, rows, cols);
            else
                orc_dequantizelinear(r.data(), x.data(), orc_type(x.get_shape().type()), s.data(),
                                     orc_type(s.get_shape().type()), cols, 1,
                                     zp.empty() ? nullptr : zp.data(), cols, 1, rows, cols);
        }
        else if(n == "unpack_int4" or n == "pack_int4")
        {
            argument x      = dense(args[0]);
            const auto& si  = x.get_shape();
            const bool unpk = n == "unpack_int4";
            int64_t axis    = unpk ? migraphx::any_cast<migraphx::op::unpack_int4>(op).axis
                                   : migraphx::any_cast<migraphx::op::pack_int4>(op).axis;
            if(axis < 0)
                axis += static_cast<int64_t>(si.ndim());
            int64_t outer = 1;
            int64_t inner = 1;
            for(int64_t i = 0; i < axis; i++)
                outer *= si.lens()[i];
            for(std::size_t i = axis + 1; i < si.ndim(); i++)
                inner *= si.lens()[i];
            const int is_signed = si.type() == shape::int8_type;
            if(unpk)
                orc_unpack_int4(reinterpret_cast<uint8_t*>(r.data()),
                                reinterpret_cast<const uint8_t*>(x.data()), is_signed, outer,
                                si.lens()[axis], inner);
            else
                orc_pack_int4(reinterpret_cast<uint8_t*>(r.data()),
                              reinterpret_cast<const uint8_t*>(x.data()), is_signed, outer,
                              out.lens()[axis], inner);
        }
        else if(n == "unpack_fp4" or n == "pack_fp4")
        {
            argument x      = dense(args[0]);
            const bool unpk = n == "unpack_fp4";
            int64_t axis    = unpk ? migraphx::any_cast<migraphx::op::unpack_fp4>(op).axis
                                   : migraphx::any_cast<migraphx::op::pack_fp4>(op).axis;
            const auto& si  = x.get_shape();
            if(axis < 0)
                axis += static_cast<int64_t>(si.ndim());
            int64_t outer = 1;
            int64_t inner = 1;
            for(int64_t i = 0; i < axis; i++)
                outer *= si.lens()[i];
            for(std::size_t i = axis + 1; i < si.ndim(); i++)
                inner *= si.lens()[i];
            if(unpk)
            {
                orc_unpack_fp4(reinterpret_cast<uint8_t*>(r.data()),
                               reinterpret_cast<const uint8_t*>(x.data()), outer, si.lens()[axis], inner);
            }
            else
            {
                // cast_to_fp4 converts its argument to float first (fp4_casts.hpp:83-85)
                argument xf{shape{shape::float_type, si.lens()}};
                orc_convert(xf.data(), orc_type(shape::float_type), x.data(), orc_type(si.type()),
                            si.elements());
                orc_pack_fp4(reinterpret_cast<uint8_t*>(r.data()),
                             reinterpret_cast<const float*>(xf.data()), outer, out.lens()[axis], inner);
            }
        }
        else if(n == "convert")
        {
            argument x = dense(args[0]);
            orc_convert(r.data(), orc_type(out.type()), x.data(), orc_type(x.get_shape().type()),
                        out.elements());
        }
        else if(n == "erf" or n == "sqrt" or n == "rsqrt" or n == "exp" or n == "tanh" or n == "neg")
        {
            argument x   = dense(args[0]);
            const int op = n == "erf" ? 0 : (n == "sqrt" ? 1 : (n == "rsqrt" ? 2 : (n == "exp" ? 3 : (n == "tanh" ? 4 : 5))));
            orc_unary_f32(op, reinterpret_cast<float*>(r.data()),
                          reinterpret_cast<const float*>(x.data()), out.elements());
        }
        else if((n == "max" or n == "min" or n == "clip" or n == "nearbyint") and out.type() == shape::float_type)
        {
            // op/max.hpp, min.hpp (std::max / std::min of the two values), op/clip.hpp:62-66
            // (std::min(std::max(lowest, x), highest)), op/nearbyint.hpp (ties to even)
            std::vector<argument> d;
            for(const auto& a : args)
                d.push_back(dense(a));
            auto* o       = reinterpret_cast<float*>(r.data());
            const auto* x = reinterpret_cast<const float*>(d[0].data());
            for(std::size_t i = 0; i < out.elements(); i++)
            {
                if(n == "nearbyint")
                    o[i] = std::nearbyint(x[i]);
                else if(n == "max")
                    o[i] = std::max(x[i], reinterpret_cast<const float*>(d[1].data())[i]);
                else if(n == "min")
                    o[i] = std::min(x[i], reinterpret_cast<const float*>(d[1].data())[i]);
                else
                    o[i] = std::min(std::max(reinterpret_cast<const float*>(d[1].data())[i], x[i]),
                                    reinterpret_cast<const float*>(d[2].data())[i]);
            }
        }
        else if((n == "reduce_max" or n == "reduce_min") and out.type() == shape::float_type)
        {
            // op/reduce_max.hpp, reduce_min.hpp over the listed axes (reduce_op.hpp:186-202): every
            // output element folds the elements that differ from it in the reduced axes only
            argument x     = dense(args[0]);
            const auto& xs = x.get_shape();
            const auto* in = reinterpret_cast<const float*>(x.data());
            auto* o        = reinterpret_cast<float*>(r.data());
            std::vector<bool> seen(out.elements(), false);
            for(std::size_t i = 0; i < xs.elements(); i++)
            {
                // the output element of input element i: reduced axes have length one
                std::size_t rem = i, oi = 0, mul = 1;
                for(std::size_t d = xs.ndim(); d-- > 0;)
                {
                    const std::size_t c = rem % xs.lens()[d];
                    rem /= xs.lens()[d];
                    if(out.lens()[d] != 1)
                    {
                        oi += c * mul;
                        mul *= out.lens()[d];
                    }
                }
                if(not seen[oi])
                {
                    o[oi]    = in[i];
                    seen[oi] = true;
                }
                else
                    o[oi] = n == "reduce_max" ? std::max(o[oi], in[i]) : std::min(o[oi], in[i]);
            }
        }
        else if(n == "reduce_mean" or n == "softmax")
        {
            // the last axis: [rows, cols, 1]
            argument x   = dense(args[0]);
            int64_t rows = 0;
            int64_t cols = 0;
            rows_cols(x.get_shape(), rows, cols);
            if(n == "reduce_mean")
            {
                // the trailing axes as one: [rows, cols] with rows = what is left of the tensor (the reduced
                // axes have length 1 in the result)
                const auto& xl = x.get_shape().lens();
                const auto& ol = out.lens();
                std::size_t first = 0;
                while(first < xl.size() and ol[first] == xl[first])
                    first++;
                for(std::size_t d = first; d < xl.size(); d++)
                {
                    if(ol[d] != 1)
                        MIGRAPHX_THROW("oracle target: reduce_mean over axes that are not the trailing ones");
                }
                rows = static_cast<int64_t>(out.elements());
                cols = rows == 0 ? 0 : static_cast<int64_t>(x.get_shape().elements()) / rows;
            }
            if(n == "reduce_mean")
                orc_reduce_mean_f32(reinterpret_cast<float*>(r.data()),
                                    reinterpret_cast<const float*>(x.data()), rows, cols, 1);
            else
                orc_softmax_f32(reinterpret_cast<float*>(r.data()),
                                reinterpret_cast<const float*>(x.data()), rows, cols, 1);
        }
        else if(n == "gather")
        {
            // axis 0
            argument t  = dense(args[0]);
            argument ix = dense(args[1]);
            auto ids    = ix.to_vector<int64_t>();
            const auto rows = static_cast<int64_t>(t.get_shape().lens()[0]);
            orc_gather(r.data(), t.data(), ids.data(), static_cast<int64_t>(ids.size()), 1, rows,
                       static_cast<int64_t>(t.get_shape().elements()) / rows,
                       static_cast<int64_t>(t.get_shape().type_size()));
        }
        else if((n == "mul" or n == "add" or n == "sub" or n == "div") and out.type() == shape::float_type)
        {
            argument x = dense(args[0]);
            argument y = dense(args[1]);
            orc_binary_f32(n == "add" ? 0 : (n == "sub" ? 1 : (n == "mul" ? 2 : 3)),
                           reinterpret_cast<float*>(r.data()), reinterpret_cast<const float*>(x.data()),
                           reinterpret_cast<const float*>(y.data()), out.elements());
        }
        else if(n == "mul" or n == "add" or n == "sub" or n == "div")
        {
            // op/binary.hpp: the plain C++ operator on the tensor's type
            migraphx::visit_type(out.type(), [&](auto t) {
                using T = decltype(t);
                auto x  = args[0].template get<T>();
                auto y  = args[1].template get<T>();
                auto o  = r.get<T>();
                for(std::size_t i = 0; i < o.size(); i++)
                {
                    if constexpr(std::is_same<T, float>{} or std::is_same<T, int32_t>{} or
                                 std::is_same<T, double>{})
                        o[i] = n == "mul" ? x[i] * y[i]
                                          : (n == "add" ? x[i] + y[i] : (n == "sub" ? x[i] - y[i] : x[i] / y[i]));
                    else if constexpr(std::is_same<T, int8_t>{} or std::is_same<T, uint8_t>{})
                    {
                        // the operands promote to int, the result converts back (wrapping)
                        const int a = x[i], b = y[i];
                        if(n == "div" and b == 0)
                            MIGRAPHX_THROW("oracle: integer division by zero");
                        const int v = n == "mul" ? a * b : (n == "add" ? a + b : (n == "sub" ? a - b : a / b));
                        o[i]        = static_cast<T>(static_cast<unsigned>(v));
                    }
                    else if constexpr(std::is_same<T, migraphx::half>{} or std::is_same<T, migraphx::bf16>{})
                    {
                        // generic_float.hpp:303-326: the operator works on floats and the result
                        // converts back to the narrow type
                        const float a = x[i], b = y[i];
                        o[i] = T(n == "mul" ? a * b : (n == "add" ? a + b : (n == "sub" ? a - b : a / b)));
                    }
                    else
                        MIGRAPHX_THROW("oracle: " + n + " on " + out.type_string());
                }
            });
        }
        else
        {
            MIGRAPHX_THROW("oracle: no implementation of " + n);
        }
        return r;
    }
};

} // namespace

migraphx::operation wrap(const migraphx::operation& op) { return migraphx::operation{cpu_op{op}}; }

void lowering::apply(migraphx::module& m) const
{
    std::vector<migraphx::instruction_ref> all;
    for(auto it = m.begin(); it != m.end(); ++it)
        all.push_back(it);
    for(auto ins : all)
    {
        const auto n = ins->name();
        if(n[0] == '@' or n == "capture" or n == "reshape" or n == "contiguous")
            continue;
        if(ins->get_operator().is_context_free())
            continue; // views
        m.replace_instruction(ins, migraphx::operation{cpu_op{ins->get_operator()}}, ins->inputs());
    }
}

std::vector<migraphx::pass> target::get_passes(migraphx::context&,
                                               const migraphx::compile_options&) const
{
    return {lowering{}, migraphx::dead_code_elimination{}};
}

} // namespace oracle

MIGRAPHX_REGISTER_TARGET(oracle::target);

// every operator of the library can come back from a saved program in its wrapped form
static const int register_wrapped_operators = [] {
    for(const auto& name : migraphx::get_operators())
    {
        if(name[0] != '@' and name.rfind("oracle::", 0) != 0)
            migraphx::register_op(migraphx::operation{oracle::wrap(migraphx::load_op(name))});
    }
    return 0;
}();
