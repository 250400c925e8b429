#include <migraphx/passes.hpp>
#include <migraphx/ops.hpp>
#include <algorithm>
#include <cmath>
#include <limits>
#include <map>
#include <set>
#include <unordered_set>

namespace migraphx {

namespace {

bool contains(const std::set<std::string>& s, const std::string& x) { return s.count(x) > 0; }

std::vector<instruction_ref> all_instructions(const module& m)
{
    std::vector<instruction_ref> r;
    for(auto it = m.begin(); it != m.end(); ++it)
        r.push_back(it);
    return r;
}

bool float_equal(double a, double b) { return a == b; }

bool all_zero(const argument& a)
{
    if(a.empty())
        return false;
    const auto v = a.to_vector<double>();
    return std::all_of(v.begin(), v.end(), [](double x) { return float_equal(x, 0); });
}

instruction_ref skip_broadcasts(instruction_ref i)
{
    while(i->name() == "broadcast" or i->name() == "multibroadcast")
        i = i->inputs().front();
    return i;
}

} // namespace

// ------------------------------------------------------- dead_code_elimination

void dead_code_elimination::apply(module& m) const
{
    if(m.size() == 0)
        return;
    std::unordered_set<const instruction*> live;
    std::vector<instruction_ref> work{std::prev(m.end())};
    while(not work.empty())
    {
        auto i = work.back();
        work.pop_back();
        if(not live.insert(&*i).second)
            continue;
        for(auto a : i->inputs())
            work.push_back(a);
    }
    // users come after their arguments: walk backwards so that users go first
    auto it = m.end();
    while(it != m.begin())
    {
        --it;
        if(live.count(&*it) > 0 or it->name() == "@param")
            continue;
        it = m.remove_instruction(it);
    }
}

// ---------------------------------------------------------------- simplify_qdq

namespace {

const std::set<std::string>& post_dq_ops()
{
    static const std::set<std::string> s = {
        "broadcast", "multibroadcast", "contiguous", "transpose", "reshape", "convert"};
    return s;
}

// dequantizelinear(x, const scale, const zp), looked for through the operators that may sit
// between it and the dot (match/dq_helpers.hpp:40-57)
instruction_ref find_dq(instruction_ref arg)
{
    while(contains(post_dq_ops(), arg->name()))
        arg = arg->inputs().front();
    return arg;
}

bool is_const_dq(instruction_ref dq)
{
    if(dq->name() != "dequantizelinear" or dq->inputs().size() != 3)
        return false;
    return skip_broadcasts(dq->inputs()[1])->can_eval() and
           skip_broadcasts(dq->inputs()[2])->can_eval();
}

std::vector<instruction_ref> get_between_ins(instruction_ref dq, instruction_ref arg)
{
    std::vector<instruction_ref> r;
    while(arg != dq)
    {
        r.push_back(arg);
        arg = arg->inputs().front();
    }
    return r;
}

// re-apply the view operators that stood between DQ and dot to the quantized tensor
// (simplify_qdq.cpp:64-82)
instruction_ref propagate_quantized_ins(module& m,
                                        instruction_ref dq,
                                        instruction_ref input,
                                        const std::vector<instruction_ref>& between,
                                        bool is_fp16_model)
{
    for(auto it = between.rbegin(); it != between.rend(); ++it)
    {
        if((*it)->name() == "convert" and is_fp16_model)
            continue;
        input = m.insert_instruction(dq, (*it)->get_operator(), input);
    }
    return input;
}

bool is_valid_qparam(instruction_ref q, const std::vector<std::size_t>& lens, std::size_t axis)
{
    return q->get_shape().elements() == 1 or q->get_shape().elements() == lens.at(axis);
}

operation qparam_broadcast_op(instruction_ref q, const std::vector<std::size_t>& lens, std::size_t axis)
{
    // one value: spread it whatever shape it came in (a scalar, or the [1] tensor of an ONNX
    // initializer)
    if(q->get_shape().scalar() or q->get_shape().elements() == 1)
        return make_op("multibroadcast", {{"out_lens", lens}});
    return make_op("broadcast", {{"out_lens", lens}, {"axis", axis}});
}

// A per-axis parameter that arrives with unit dimensions around its axis (the ONNX parsers
// unsqueeze a vector to the tensor's rank before they broadcast it) as the vector `broadcast`
// takes.  The reference leaves this to the passes that run in front of simplify_qdq on its
// targets; here the pass does it itself.
instruction_ref as_vector(module& m, instruction_ref pos, instruction_ref q)
{
    const auto& s = q->get_shape();
    if(s.scalar() or s.ndim() <= 1)
        return q;
    if(not s.standard())
        q = m.insert_instruction(pos, make_op("contiguous"), q);
    return m.insert_instruction(pos, make_op("reshape", {{"dims", {static_cast<int64_t>(s.elements())}}}), q);
}

bool is_symmetric_zero_point(instruction_ref zp)
{
    if(not zp->can_eval())
        return false;
    return all_zero(zp->eval());
}

bool is_quantized_type(shape::type_t t)
{
    return t == shape::int8_type or t == shape::fp8e4m3fn_type or t == shape::fp8e4m3fnuz_type or
           t == shape::fp8e5m2_type or t == shape::fp8e5m2fnuz_type;
}

// simplify_qdq.cpp:126-289: the dot branch and the convolution branch (:171-222)
void find_quantizable_dot(module& m, instruction_ref qop)
{
    auto dq1 = find_dq(qop->inputs()[0]);
    auto dq2 = find_dq(qop->inputs()[1]);
    if(not is_const_dq(dq1) or not is_const_dq(dq2))
        return;
    auto scale1 = skip_broadcasts(dq1->inputs()[1]);
    auto zp1    = skip_broadcasts(dq1->inputs()[2]);
    auto scale2 = skip_broadcasts(dq2->inputs()[1]);
    auto zp2    = skip_broadcasts(dq2->inputs()[2]);

    bool is_fp16_model = false;
    if(dq1->get_shape().type() != qop->get_shape().type() and
       qop->get_shape().type() == shape::half_type)
        is_fp16_model = true;

    auto qop_args = qop->inputs();
    auto between0 = get_between_ins(dq1, qop_args[0]);
    auto between1 = get_between_ins(dq2, qop_args[1]);
    qop_args[0]   = propagate_quantized_ins(m, dq1, dq1->inputs().front(), between0, is_fp16_model);
    qop_args[1]   = propagate_quantized_ins(m, dq2, dq2->inputs().front(), between1, is_fp16_model);
    auto arg1_lens = qop_args[0]->get_shape().lens();
    auto arg2_lens = qop_args[1]->get_shape().lens();

    // only int8 and fp8 tensors are rewritten; uint8 Q/DQ stays as it is (:157-165)
    if(not is_quantized_type(dq1->inputs().front()->get_shape().type()) or
       not is_quantized_type(dq2->inputs().front()->get_shape().type()))
        return;

    if(qop->name() == "convolution")
    {
        // simplify_qdq.cpp:171-222: the input may only carry one scale and zero point, the
        // weights one per output channel (axis 0 of the weights, axis 1 of the result)
        const auto conv_val = qop->get_operator().to_value();
        auto qconv          = m.insert_instruction(qop, make_op("quant_convolution", conv_val), qop_args);
        auto conv_lens      = qconv->get_shape().lens();
        if(not(scale1->get_shape().elements() == 1 and zp1->get_shape().elements() == 1 and
               is_valid_qparam(scale2, arg2_lens, 0) and is_valid_qparam(zp2, arg2_lens, 0)))
            return;
        scale2 = as_vector(m, qop, scale2);
        zp2    = as_vector(m, qop, zp2);
        auto s1 = m.insert_instruction(qop, qparam_broadcast_op(scale1, conv_lens, 1), scale1);
        auto s2 = m.insert_instruction(qop, qparam_broadcast_op(scale2, conv_lens, 1), scale2);
        auto conv_scale = m.insert_instruction(qop, make_op("mul"), s1, s2);
        auto zero = m.add_literal(literal{shape{qconv->get_shape().type()}, std::vector<int>{0}});
        auto conv_zp =
            m.insert_instruction(qop, make_op("multibroadcast", {{"out_lens", conv_lens}}), zero);
        auto in_zp_bc = m.insert_instruction(qop, qparam_broadcast_op(zp1, arg1_lens, 1), zp1);
        auto w_zp_bc  = m.insert_instruction(qop, qparam_broadcast_op(zp2, arg2_lens, 0), zp2);
        const bool s1z = is_symmetric_zero_point(zp1);
        const bool s2z = is_symmetric_zero_point(zp2);
        if(not s1z)
        {
            auto t  = m.insert_instruction(qop, make_op("quant_convolution", conv_val), in_zp_bc, qop_args[1]);
            conv_zp = m.insert_instruction(qop, make_op("add"), conv_zp, t);
        }
        if(not s2z)
        {
            auto t  = m.insert_instruction(qop, make_op("quant_convolution", conv_val), qop_args[0], w_zp_bc);
            conv_zp = m.insert_instruction(qop, make_op("add"), conv_zp, t);
        }
        if(not s1z and not s2z)
        {
            auto t  = m.insert_instruction(qop, make_op("quant_convolution", conv_val), in_zp_bc, w_zp_bc);
            conv_zp = m.insert_instruction(qop, make_op("sub"), conv_zp, t);
        }
        auto r = m.insert_instruction(qop, make_op("dequantizelinear"), qconv, conv_scale, conv_zp);
        if(is_fp16_model)
            r = m.insert_instruction(qop, make_op("convert", {{"target_type", shape::half_type}}), r);
        m.replace_instruction(qop, r);
        return;
    }

    auto dq       = m.insert_instruction(qop, make_op("quant_dot"), qop_args);
    auto out_lens = dq->get_shape().lens();
    const std::size_t nd = out_lens.size();
    // valid quantization axes: M for the first input, N for the second (:232-238)
    if(not(is_valid_qparam(scale1, out_lens, nd - 2) and is_valid_qparam(zp1, out_lens, nd - 2) and
           is_valid_qparam(scale2, out_lens, nd - 1) and is_valid_qparam(zp2, out_lens, nd - 1)))
        return;
    scale1 = as_vector(m, qop, scale1);
    zp1    = as_vector(m, qop, zp1);
    scale2 = as_vector(m, qop, scale2);
    zp2    = as_vector(m, qop, zp2);

    auto s1_bcast = m.insert_instruction(qop, qparam_broadcast_op(scale1, out_lens, nd - 2), scale1);
    auto s2_bcast = m.insert_instruction(qop, qparam_broadcast_op(scale2, out_lens, nd - 1), scale2);
    auto out_scale = m.insert_instruction(qop, make_op("mul"), s1_bcast, s2_bcast);

    // zero-point terms: 0 [+ zp1*B] [+ A*zp2] [- zp1*zp2] (:250-279)
    auto zero_lit = m.add_literal(literal{shape{dq->get_shape().type()}, std::vector<int>{0}});
    auto out_zp =
        m.insert_instruction(qop, make_op("multibroadcast", {{"out_lens", out_lens}}), zero_lit);
    auto zp1_bc =
        m.insert_instruction(qop, qparam_broadcast_op(zp1, arg1_lens, arg1_lens.size() - 2), zp1);
    auto zp2_bc =
        m.insert_instruction(qop, qparam_broadcast_op(zp2, arg2_lens, arg2_lens.size() - 1), zp2);
    const bool sym1 = is_symmetric_zero_point(zp1);
    const bool sym2 = is_symmetric_zero_point(zp2);
    if(not sym1)
    {
        auto t = m.insert_instruction(qop, make_op("quant_dot"), zp1_bc, qop_args[1]);
        out_zp = m.insert_instruction(qop, make_op("add"), out_zp, t);
    }
    if(not sym2)
    {
        auto t = m.insert_instruction(qop, make_op("quant_dot"), qop_args[0], zp2_bc);
        out_zp = m.insert_instruction(qop, make_op("add"), out_zp, t);
    }
    if(not sym1 and not sym2)
    {
        auto t = m.insert_instruction(qop, make_op("quant_dot"), zp1_bc, zp2_bc);
        out_zp = m.insert_instruction(qop, make_op("sub"), out_zp, t);
    }

    dq = m.insert_instruction(qop, make_op("dequantizelinear"), dq, out_scale, out_zp);
    if(is_fp16_model)
        dq = m.insert_instruction(qop, make_op("convert", {{"target_type", shape::half_type}}), dq);
    m.replace_instruction(qop, dq);
}

// simplify_qdq.cpp:290-357: block quantization of the MX types.  Both operands of the dot come
// (through view operators) from a two-input dequantizelinear whose scale, behind its broadcasts,
// is neither a scalar nor one-dimensional, i.e. has the operand's own rank: one scale per block,
// spread over the elements.  The dot becomes quant_dot(a, b, scale_a, scale_b), the operators that
// stood between each DQ and the dot re-applied to its tensor and to its scales alike.
bool is_block_dq(instruction_ref dq)
{
    if(dq->name() != "dequantizelinear" or dq->inputs().size() != 2)
        return false;
    auto scale = skip_broadcasts(dq->inputs()[1]);
    return not scale->get_shape().scalar() and scale->get_shape().ndim() != 1;
}

void find_mx_quantizable_dot(module& m, instruction_ref qop)
{
    auto dq1 = find_dq(qop->inputs()[0]);
    auto dq2 = find_dq(qop->inputs()[1]);
    if(not is_block_dq(dq1) or not is_block_dq(dq2))
        return;
    bool is_fp16_model = false;
    if(dq1->get_shape().type() != qop->get_shape().type() and
       qop->get_shape().type() == shape::half_type)
        is_fp16_model = true;
    auto qop_args = qop->inputs();
    auto between0 = get_between_ins(dq1, qop_args[0]);
    auto between1 = get_between_ins(dq2, qop_args[1]);
    qop_args[0]   = propagate_quantized_ins(m, dq1, dq1->inputs().front(), between0, is_fp16_model);
    qop_args[1]   = propagate_quantized_ins(m, dq2, dq2->inputs().front(), between1, is_fp16_model);
    qop_args.push_back(propagate_quantized_ins(m, dq1, dq1->inputs()[1], between0, is_fp16_model));
    qop_args.push_back(propagate_quantized_ins(m, dq2, dq2->inputs()[1], between1, is_fp16_model));
    m.replace_instruction(qop, make_op("quant_dot"), qop_args);
}

// simplify_qdq.cpp:360-394
bool compare_literals(instruction_ref a, instruction_ref b)
{
    a      = skip_broadcasts(a);
    b      = skip_broadcasts(b);
    auto x = a->eval();
    auto y = b->eval();
    if(x.empty() or y.empty())
        return false;
    if(x.get_shape().type() != y.get_shape().type())
        return false;
    auto vx = x.to_vector<double>();
    auto vy = y.to_vector<double>();
    if(x.get_shape() == y.get_shape() and vx == vy)
        return true;
    auto same = [&](double v) {
        return float_equal(v, vx.front()) or (std::isinf(vx.front()) and std::isinf(v));
    };
    return std::all_of(vx.begin() + 1, vx.end(), same) and std::all_of(vy.begin(), vy.end(), same);
}

bool is_same_value(instruction_ref a, instruction_ref b) { return a == b or compare_literals(a, b); }

bool is_same_scale_zero(instruction_ref a, instruction_ref b)
{
    if(a->inputs().size() != b->inputs().size())
        return false;
    if(not is_same_value(a->inputs().at(1), b->inputs().at(1)))
        return false;
    if(a->inputs().size() == 2)
        return true;
    return is_same_value(a->inputs().at(2), b->inputs().at(2));
}

// simplify_qdq.cpp:498-533
void remove_qdq_pairs(module& m)
{
    static const std::set<std::string> skip_set = {"broadcast", "slice", "reshape", "pad"};
    for(auto dq : all_instructions(m))
    {
        if(dq->name() != "dequantizelinear")
            continue;
        auto q = dq->inputs().front();
        while(contains(skip_set, q->name()) and q->inputs().size() == 1)
            q = q->inputs().front();
        if(q->name() != "quantizelinear")
            continue;
        if(not is_same_scale_zero(dq, q))
            continue;
        auto users = dq->outputs();
        for(auto u : users)
            instruction::replace_argument(u, dq, q->inputs().front());
    }
}

// simplify_qdq.cpp:574-594
void remove_zero_point(module& m)
{
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "dequantizelinear" or ins->inputs().size() != 3)
            continue;
        auto zp = ins->inputs()[2];
        if(not zp->can_eval() or not all_zero(zp->eval()))
            continue;
        m.replace_instruction(ins, ins->get_operator(), ins->inputs()[0], ins->inputs()[1]);
    }
}

// simplify_qdq.cpp:596-620
void remove_zero_scales(module& m)
{
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "dequantizelinear" or ins->inputs().size() < 2)
            continue;
        auto scale = ins->inputs()[1];
        if(not scale->can_eval() or not all_zero(scale->eval()))
            continue;
        auto zero = m.add_literal(literal{shape{ins->get_shape().type()}, std::vector<int>{0}});
        auto bc   = m.insert_instruction(
            ins, make_op("multibroadcast", {{"out_lens", ins->get_shape().lens()}}), zero);
        m.replace_instruction(ins, bc);
    }
}

// simplify_qdq.cpp:439-453, :623-640: a quantizelinear fed (through view operators) by
// unpack_int4 holds 4-bit data, so it is stored packed
void add_int4_pack_unpack_pair(module& m)
{
    static const std::set<std::string> ign = {
        "unsqueeze", "broadcast", "multibroadcast", "contiguous", "transpose", "reshape", "convert"};
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "dequantizelinear")
            continue;
        auto inputs = ins->inputs();
        for(auto inp : inputs)
        {
            if(inp->name() != "quantizelinear")
                continue;
            const bool int4 = std::any_of(inp->inputs().begin(), inp->inputs().end(), [](auto i) {
                while(contains(ign, i->name()))
                    i = i->inputs()[0];
                return i->name() == "unpack_int4";
            });
            if(not int4)
                continue;
            auto pk   = m.insert_instruction(ins, make_op("pack_int4"), inp);
            auto unpk = m.insert_instruction(ins, make_op("unpack_int4"), pk);
            instruction::replace_argument(ins, inp, unpk);
        }
    }
}

} // namespace

void simplify_qdq::apply(module& m) const
{
    remove_zero_scales(m);
    if(remove_qdq_only)
    {
        remove_qdq_pairs(m);
        return;
    }
    add_int4_pack_unpack_pair(m);
    for(auto ins : all_instructions(m))
    {
        if(ins->name() == "dot" or ins->name() == "convolution")
            find_quantizable_dot(m, ins);
    }
    dead_code_elimination{}.apply(m);
    if(use_mx_quant)
    {
        for(auto ins : all_instructions(m))
        {
            if(ins->name() == "dot")
                find_mx_quantizable_dot(m, ins);
        }
        dead_code_elimination{}.apply(m);
    }
    remove_qdq_pairs(m);
    dead_code_elimination{}.apply(m);
    remove_zero_point(m);
}

// ---------------------------------------------------------------- quantize 8 bits

namespace {
const std::set<shape::type_t>& quantizable_types()
{
    static const std::set<shape::type_t> s = {
        shape::float_type, shape::double_type, shape::half_type};
    return s;
}
} // namespace

void capture_arguments_pass::apply(module& m) const
{
    if(param_index == nullptr)
        MIGRAPHX_THROW("capture_arguments: no parameter counter");
    for(auto ins : all_instructions(m))
    {
        if(ins_names.count(ins->name()) == 0 or ins->name() == "convert")
            continue;
        std::vector<instruction_ref> new_args;
        for(auto input : ins->inputs())
        {
            if(quantizable_types().count(input->get_shape().type()) > 0)
            {
                op::capture c;
                c.ins_index = (*param_index)++;
                c.f         = f;
                new_args.push_back(m.insert_instruction(ins, operation{c}, input));
            }
            else
            {
                new_args.push_back(input);
            }
        }
        m.replace_instruction(ins, ins->get_operator(), new_args);
    }
}

void quantize_8bits_pass::apply(module& m) const
{
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "capture")
            continue;
        const auto index = any_cast<op::capture>(ins->get_operator()).ins_index;
        const auto param = quant_params.at(index);
        auto input       = ins->inputs().front();
        const auto s     = input->get_shape();
        if(quantizable_types().count(s.type()) == 0 or s.type() == precision)
            continue;
        auto zero_point = m.add_literal(literal{shape{precision}, std::vector<float>{param.second}});
        // the Q/DQ scale is the inverse of the calibrated multiplier, kept within the tensor
        // type's [epsilon, max] (quantize_8bits.cpp:73-83)
        float inverted_scale = 1.0f / param.first;
        float epsilon        = 0.0f;
        float max_val        = std::numeric_limits<float>::max();
        visit_type(s.type(), [&](auto x) {
            using T = decltype(x);
            epsilon = static_cast<float>(std::numeric_limits<T>::epsilon());
            max_val = static_cast<float>(std::numeric_limits<T>::max());
        });
        inverted_scale = std::max(epsilon, std::min(max_val, inverted_scale));
        auto scale     = m.add_literal(literal{shape{s.type()}, std::vector<float>{inverted_scale}});
        auto scale_bc =
            m.insert_instruction(ins, make_op("multibroadcast", {{"out_lens", s.lens()}}), scale);
        auto zp_bc = m.insert_instruction(
            ins, make_op("multibroadcast", {{"out_lens", s.lens()}}), zero_point);
        auto q  = m.insert_instruction(ins, make_op("quantizelinear"), input, scale_bc, zp_bc);
        auto dq = m.insert_instruction(ins, make_op("dequantizelinear"), q, scale_bc, zp_bc);
        m.replace_instruction(ins, dq);
    }
}

namespace {

void quantize_8bits(program& prog,
                    const target& t,
                    shape::type_t precision,
                    const std::vector<parameter_map>& calibration,
                    const std::unordered_set<std::string>& ins_names)
{
    auto params   = std::make_shared<std::vector<std::pair<float, float>>>();
    auto max_abs  = std::make_shared<std::vector<float>>();
    static const std::map<shape::type_t, float> ranges = {{shape::int8_type, 127.0f},
                                                          {shape::fp8e4m3fnuz_type, 240.0f},
                                                          {shape::fp8e4m3fn_type, 448.0f}};
    const float quantized_range = ranges.at(precision);
    // scale = range / max|x| over all calibration runs; the shift stays 0 (quantization.cpp:101-130)
    auto calc = [=](std::size_t index, std::vector<argument> args) {
        argument host = t.copy_from(args.front());
        auto v        = host.to_vector<float>();
        float m       = 0.0f;
        for(float x : v)
            m = std::max(m, std::fabs(x));
        max_abs->at(index)   = std::max(max_abs->at(index), m);
        std::pair<float, float> p{64.0f, 0.0f};
        p.first           = float_equal(max_abs->at(index), 0.0f) ? 1.0f : quantized_range / max_abs->at(index);
        params->at(index) = p;
    };

    std::size_t param_num = 0;
    run_passes(prog, {capture_arguments_pass{ins_names, calc, &param_num}});
    params->resize(param_num, std::pair<float, float>(64.0f, 0.0f));
    max_abs->resize(param_num, 0.0f);

    program capture_prog = prog;
    capture_prog.compile(t);
    for(const auto& arg : calibration)
    {
        parameter_map pm;
        for(const auto& x : capture_prog.get_parameter_shapes())
        {
            auto it = arg.find(x.first);
            pm[x.first] = it != arg.end() ? t.copy_to(it->second) : t.allocate(x.second);
        }
        capture_prog.eval(pm);
        capture_prog.finish();
    }
    run_passes(prog, {quantize_8bits_pass{precision, *params}, dead_code_elimination{}});
}

} // namespace

void quantize_int8(program& prog,
                   const target& t,
                   const std::vector<parameter_map>& calibration,
                   const std::unordered_set<std::string>& ins_names)
{
    const std::unordered_set<std::string> op_names = {"convolution", "dot"};
    if(op_names != ins_names)
        MIGRAPHX_THROW("QUANTIZE_INT8: only support DOT and CONVOLUTION operation");
    quantize_8bits(prog, t, shape::int8_type, calibration, ins_names);
}

void quantize_fp8(program& prog, const target& t, const std::vector<parameter_map>& calibration)
{
    std::unordered_set<std::string> names;
    for(auto ins : all_instructions(*prog.get_main_module()))
    {
        if(ins->name() == "convert" or ins->name()[0] == '@')
            continue;
        names.insert(ins->name());
    }
    quantize_8bits(prog, t, shape::fp8e4m3fn_type, calibration, names);
}

// ---------------------------------------------------------------- quantize int4

void quantize_int4_pass::apply(module& m) const
{
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "dot" or ins->inputs().empty())
            continue;
        const auto out_type = ins->get_shape().type();
        auto inputs         = ins->inputs();
        for(auto& inp : inputs)
        {
            const auto sh = inp->get_shape();
            if(sh.broadcasted())
                continue;
            if(sh.type() != shape::float_type and sh.type() != shape::half_type)
                continue;
            const auto lens = sh.lens();
            if(lens.back() % 2 != 0)
                continue; // the packed axis must be even
            if(not inp->can_eval())
                continue;
            auto val = inp->eval().to_vector<float>();
            if(val.empty())
                continue;
            // per-tensor affine parameters over [min(0, min), max(0, max)] mapped to [0, 15]
            float lo = std::min(0.0f, *std::min_element(val.begin(), val.end()));
            float hi = std::max(0.0f, *std::max_element(val.begin(), val.end()));
            const float fscale4 = (hi - lo) / 15;
            const int zp4       = float_equal(fscale4, 0) ? 0 : static_cast<int>(std::round(-lo / fscale4));
            auto bcast          = make_op("multibroadcast", {{"out_lens", lens}});
            auto scale = m.add_literal(literal{shape{out_type}, std::vector<float>{fscale4}});
            scale      = m.insert_instruction(ins, bcast, scale);
            auto zp    = m.add_literal(literal{shape{shape::uint8_type}, std::vector<int>{zp4}});
            zp         = m.insert_instruction(ins, bcast, zp);
            auto q     = m.insert_instruction(ins, make_op("quantizelinear"), inp, scale, zp);
            auto pk    = m.insert_instruction(ins, make_op("pack_int4", {{"axis", -1}}), q);
            auto unpk  = m.insert_instruction(ins, make_op("unpack_int4", {{"axis", -1}}), pk);
            auto dq_scale = m.add_literal(literal{shape{out_type}, std::vector<float>{fscale4}});
            dq_scale      = m.insert_instruction(ins, bcast, dq_scale);
            auto dq_zp = m.add_literal(literal{shape{shape::uint8_type}, std::vector<int>{zp4}});
            dq_zp      = m.insert_instruction(ins, bcast, dq_zp);
            inp = m.insert_instruction(ins, make_op("dequantizelinear"), unpk, dq_scale, dq_zp);
        }
        auto converted = m.insert_instruction(ins, ins->get_operator(), inputs);
        m.replace_instruction(ins, converted);
    }
}

void quantize_int4_weights(program& prog) { run_passes(prog, {quantize_int4_pass{}}); }

// ---------------------------------------------------------------- MatMulNBits

namespace op {
namespace builder {

namespace {

// parse_matmulnbits.cpp:128-138
instruction_ref unpack(module& m, std::size_t n, std::size_t dim1, instruction_ref x)
{
    x = m.add_instruction(make_op("reshape", {{"dims", {static_cast<int64_t>(n), -1}}}), x);
    x = m.add_instruction(make_op("unpack_int4"), x);
    if(x->get_shape().lens()[1] > dim1)
        x = m.add_instruction(
            make_op("slice", {{"axes", {1}}, {"starts", {0}}, {"ends", {dim1}}}), x);
    return x;
}

// parse_matmulnbits.cpp:140-158: repeat every per-block value block_size times along K
instruction_ref
blockwise_arg(module& m, std::size_t n, std::size_t k, std::size_t block_size, instruction_ref x)
{
    x            = m.add_instruction(make_op("unsqueeze", {{"axes", {2}}}), x);
    auto bc_lens = x->get_shape().lens();
    bc_lens[2]   = block_size;
    x            = m.add_instruction(make_op("multibroadcast", {{"out_lens", bc_lens}}), x);
    x = m.add_instruction(make_op("reshape", {{"dims", {static_cast<int64_t>(n), -1}}}), x);
    if(x->get_shape().lens()[1] > k) // runt block
        x = m.add_instruction(make_op("slice", {{"axes", {1}}, {"starts", {0}}, {"ends", {k}}}), x);
    return x;
}

} // namespace

instruction_ref matmulnbits(module& m,
                            instruction_ref a,
                            instruction_ref b,
                            instruction_ref scales,
                            instruction_ref zp,
                            std::size_t n,
                            std::size_t k,
                            std::size_t block_size)
{
    if(block_size < 16 or (block_size & (block_size - 1)) != 0)
        MIGRAPHX_THROW("MatMulNBits: block_size must be a power of 2 and >=16, actual value " +
                       std::to_string(block_size));
    const std::size_t n_blocks = (k + block_size - 1) / block_size;
    const std::size_t blob     = block_size / 2;
    if(b->get_shape().lens() != std::vector<std::size_t>{n, n_blocks, blob})
        MIGRAPHX_THROW("MatMulNBits: Input B does not match expected dims");
    if(scales->get_shape().elements() != n * n_blocks)
        MIGRAPHX_THROW("MatMulNBits: Input scales does not match expected dims");
    const bool has_zp = zp != m.end();
    if(has_zp and zp->get_shape().lens() != std::vector<std::size_t>{n * ((n_blocks + 1) / 2)})
        MIGRAPHX_THROW("MatMulNBits: Input zero_points does not match expected dims");

    auto bq = unpack(m, n, k, b);
    auto sc = m.add_instruction(make_op("reshape", {{"dims", {static_cast<int64_t>(n), -1}}}), scales);
    sc      = blockwise_arg(m, n, k, block_size, sc);
    instruction_ref z;
    if(has_zp)
    {
        z = unpack(m, n, n_blocks, zp);
        z = blockwise_arg(m, n, k, block_size, z);
    }
    else
    {
        z = m.add_literal(literal{shape{shape::uint8_type, {1}}, std::vector<int>{8}});
        z = m.add_instruction(make_op("multibroadcast", {{"out_lens", bq->get_shape().lens()}}), z);
    }
    auto dq = m.add_instruction(make_op("dequantizelinear"), bq, sc, z);
    auto bt = m.add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), dq);
    // numpy matmul rules for A (the reference's matmul helper, src/onnx/parse_matmul.cpp): a vector
    // is a one-row matrix, leading dimensions of A broadcast over B
    const auto a_lens = a->get_shape().lens();
    if(a_lens.size() == 1)
    {
        auto a2 = m.add_instruction(make_op("unsqueeze", {{"axes", {0}}}), a);
        auto d  = m.add_instruction(make_op("dot"), a2, bt);
        return m.add_instruction(make_op("squeeze", {{"axes", {0}}}), d);
    }
    if(a_lens.size() > 2)
    {
        std::vector<std::size_t> bl(a_lens.begin(), a_lens.end() - 2);
        bl.push_back(k);
        bl.push_back(n);
        bt = m.add_instruction(make_op("multibroadcast", {{"out_lens", bl}}), bt);
    }
    return m.add_instruction(make_op("dot"), a, bt);
}

} // namespace builder
} // namespace op

} // namespace migraphx
