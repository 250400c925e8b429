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

// ---- a product operand that comes out of a dequantizelinear ------------------------------------
//
// Between a dot / convolution argument and the dequantizelinear that made it there may stand
// operators that only re-label or re-type the tensor (match/dq_helpers.hpp:40-57 lists them).
// The rewrite moves the product in front of the dequantization, so those operators have to be
// applied to the quantized tensor instead (simplify_qdq.cpp:49-82).
struct dequantized_operand
{
    instruction_ref dq;
    std::vector<instruction_ref> views; // what stood between, the one next to dq first

    static bool passes_through(const std::string& name)
    {
        static const std::set<std::string> names = {
            "broadcast", "multibroadcast", "contiguous", "transpose", "reshape", "convert"};
        return names.count(name) > 0;
    }

    static dequantized_operand behind(instruction_ref arg)
    {
        dequantized_operand r;
        while(passes_through(arg->name()))
        {
            r.views.insert(r.views.begin(), arg);
            arg = arg->inputs().front();
        }
        r.dq = arg;
        return r;
    }

    bool is_dq() const { return dq->name() == "dequantizelinear"; }
    instruction_ref tensor() const { return dq->inputs()[0]; }
    instruction_ref scale() const { return skip_broadcasts(dq->inputs()[1]); }
    instruction_ref zero_point() const { return skip_broadcasts(dq->inputs()[2]); }

    // scale and zero point both present and known at compile time
    bool constant_parameters() const
    {
        return is_dq() and dq->inputs().size() == 3 and scale()->can_eval() and zero_point()->can_eval();
    }

    // MX block quantization: no zero point, and a scale of the tensor's own rank (one value per
    // block, spread over the block's elements by the broadcasts in front of it)
    bool block_scaled() const
    {
        if(not is_dq() or dq->inputs().size() != 2)
            return false;
        const auto& s = scale()->get_shape();
        return not s.scalar() and s.ndim() != 1;
    }

    // x with the operand's view operators on top, inserted in front of the dequantizelinear; a
    // `convert` among them is dropped when the product's own type says the model runs in half
    instruction_ref with_views(module& m, instruction_ref x, bool half_model) const
    {
        for(auto v : views)
        {
            if(half_model and v->name() == "convert")
                continue;
            x = m.insert_instruction(dq, v->get_operator(), x);
        }
        return x;
    }
};

// the product's result is half while the dequantized operands are not: an fp16 model whose Q/DQ
// pairs were inserted in float; the rewritten product converts its result back (:283-287)
bool runs_in_half(instruction_ref product, const dequantized_operand& a)
{
    return product->get_shape().type() == shape::half_type and a.dq->get_shape().type() != shape::half_type;
}

bool is_quantized_type(shape::type_t t)
{
    return t == shape::int8_type or t == shape::fp8e4m3fn_type or t == shape::fp8e4m3fnuz_type or
           t == shape::fp8e5m2_type or t == shape::fp8e5m2fnuz_type;
}

bool evaluates_to_zero(instruction_ref x) { return x->can_eval() and all_zero(x->eval()); }

// one value, or one value per index of `axis`
instruction_ref spread(module& m, instruction_ref pos, instruction_ref q, const std::vector<std::size_t>& lens,
                       std::size_t axis)
{
    // a single value is spread whatever shape it came in (a scalar, or the [1] tensor of an
    // ONNX initializer)
    if(q->get_shape().scalar() or q->get_shape().elements() == 1)
        return m.insert_instruction(pos, make_op("multibroadcast", {{"out_lens", lens}}), q);
    return m.insert_instruction(pos, make_op("broadcast", {{"out_lens", lens}, {"axis", axis}}), q);
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

// ---- dot / convolution of two dequantized tensors -> quantized product + one dequantizelinear --
//
// simplify_qdq.cpp:128-289.  dot and convolution differ only in where a per-axis parameter of
// each operand runs: along M / N of a dot's result and operands (:232-238), along the output
// channels for a convolution's weights, while a convolution's input may carry one scale and one
// zero point only (:171-195).  With x = sa (qa - za), w = sb (qb - zb):
//   x * w = sa sb [ qa*qb - za*qb - qa*zb + za*zb ]
// so the result is dequantizelinear(qa*qb, scale = sa sb, zero point = za*qb + qa*zb - za*zb),
// each `*` the quantized product itself and the zero-point terms present only for non-zero
// zero points (:196-222, :250-279).
struct product_axes
{
    std::size_t in_result[2];  // axis of the result the parameters of operand 0 / 1 follow
    std::size_t in_operand[2]; // the same axis in the operand itself
    bool per_axis[2];          // may the operand carry one parameter per index at all
};

void quantize_product(module& m, instruction_ref product)
{
    const dequantized_operand side[2] = {dequantized_operand::behind(product->inputs()[0]),
                                         dequantized_operand::behind(product->inputs()[1])};
    if(not side[0].constant_parameters() or not side[1].constant_parameters())
        return;
    const bool half_model = runs_in_half(product, side[0]);
    const bool is_conv    = product->name() == "convolution";

    instruction_ref q[2], scale[2], zp[2];
    for(int i = 0; i < 2; i++)
    {
        q[i]     = side[i].with_views(m, side[i].tensor(), half_model);
        scale[i] = side[i].scale();
        zp[i]    = side[i].zero_point();
    }
    // only int8 and fp8 tensors are rewritten; uint8 Q/DQ stays as it is (:157-165)
    if(not is_quantized_type(side[0].tensor()->get_shape().type()) or
       not is_quantized_type(side[1].tensor()->get_shape().type()))
        return;

    const operation qop = is_conv ? make_op("quant_convolution", product->get_operator().to_value())
                                  : make_op("quant_dot");
    auto multiply       = [&](instruction_ref x, instruction_ref w) { return m.insert_instruction(product, qop, x, w); };
    auto acc            = multiply(q[0], q[1]);
    const auto lens     = acc->get_shape().lens();
    const std::vector<std::size_t> operand_lens[2] = {q[0]->get_shape().lens(), q[1]->get_shape().lens()};
    const std::size_t nd = lens.size();
    const product_axes ax =
        is_conv ? product_axes{{1, 1}, {1, 0}, {false, true}}
                : product_axes{{nd - 2, nd - 1}, {operand_lens[0].size() - 2, operand_lens[1].size() - 1}, {true, true}};
    for(int i = 0; i < 2; i++)
    {
        for(auto p : {scale[i], zp[i]})
        {
            const auto n = p->get_shape().elements();
            if(n != 1 and not(ax.per_axis[i] and n == lens.at(ax.in_result[i])))
                return; // parameters along another axis: the graph stays as it was
        }
    }
    for(int i = 0; i < 2; i++)
    {
        if(not ax.per_axis[i])
            continue;
        scale[i] = as_vector(m, product, scale[i]);
        zp[i]    = as_vector(m, product, zp[i]);
    }

    auto sa        = spread(m, product, scale[0], lens, ax.in_result[0]);
    auto sb        = spread(m, product, scale[1], lens, ax.in_result[1]);
    auto out_scale = m.insert_instruction(product, make_op("mul"), sa, sb);

    auto zero      = m.add_literal(literal{shape{acc->get_shape().type()}, std::vector<int>{0}});
    auto shift     = m.insert_instruction(product, make_op("multibroadcast", {{"out_lens", lens}}), zero);
    auto za        = spread(m, product, zp[0], operand_lens[0], ax.in_operand[0]);
    auto zb        = spread(m, product, zp[1], operand_lens[1], ax.in_operand[1]);
    const bool has_za = not evaluates_to_zero(zp[0]);
    const bool has_zb = not evaluates_to_zero(zp[1]);
    if(has_za)
        shift = m.insert_instruction(product, make_op("add"), shift, multiply(za, q[1]));
    if(has_zb)
        shift = m.insert_instruction(product, make_op("add"), shift, multiply(q[0], zb));
    if(has_za and has_zb)
        shift = m.insert_instruction(product, make_op("sub"), shift, multiply(za, zb));

    auto result = m.insert_instruction(product, make_op("dequantizelinear"), acc, out_scale, shift);
    if(half_model)
        result = m.insert_instruction(product, make_op("convert", {{"target_type", shape::half_type}}), result);
    m.replace_instruction(product, result);
}

// simplify_qdq.cpp:290-357: block quantization of the MX types.  Both operands of the dot come
// (through view operators) from a two-input dequantizelinear with one scale per block.  The dot
// becomes quant_dot(a, b, scale_a, scale_b); what stood between each dequantizelinear and the dot
// is applied to its tensor and to its scales alike.
void quantize_block_scaled_dot(module& m, instruction_ref dot)
{
    const auto a = dequantized_operand::behind(dot->inputs()[0]);
    const auto b = dequantized_operand::behind(dot->inputs()[1]);
    if(not a.block_scaled() or not b.block_scaled())
        return;
    const bool half_model = runs_in_half(dot, a);
    std::vector<instruction_ref> args;
    args.push_back(a.with_views(m, a.tensor(), half_model));
    args.push_back(b.with_views(m, b.tensor(), half_model));
    args.push_back(a.with_views(m, a.dq->inputs()[1], half_model));
    args.push_back(b.with_views(m, b.dq->inputs()[1], half_model));
    m.replace_instruction(dot, make_op("quant_dot"), args);
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
            quantize_product(m, ins);
    }
    dead_code_elimination{}.apply(m);
    if(use_mx_quant)
    {
        for(auto ins : all_instructions(m))
        {
            if(ins->name() == "dot")
                quantize_block_scaled_dot(m, ins);
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

namespace {

// The scale a quantizelinear / dequantizelinear pair carries is the inverse of the calibrated
// multiplier, held inside what the tensor's own type can represent: at least its epsilon, at
// most its largest finite value (quantize_8bits.cpp:73-83).
float qdq_scale_for(float multiplier, shape::type_t tensor_type)
{
    float smallest = 0.0f;
    float largest  = std::numeric_limits<float>::max();
    visit_type(tensor_type, [&](auto tag) {
        using limits = std::numeric_limits<decltype(tag)>;
        smallest     = static_cast<float>(limits::epsilon());
        largest      = static_cast<float>(limits::max());
    });
    return std::clamp(1.0f / multiplier, smallest, largest);
}

} // namespace

// Every `capture` that marks a float tensor is replaced by quantizelinear -> dequantizelinear with
// that tensor's calibrated parameters (quantize_8bits.cpp:52-96); simplify_qdq later moves the
// products in front of the dequantizations.
void quantize_8bits_pass::apply(module& m) const
{
    for(auto marker : all_instructions(m))
    {
        if(marker->name() != "capture")
            continue;
        auto x           = marker->inputs().front();
        const auto& xs   = x->get_shape();
        if(quantizable_types().count(xs.type()) == 0 or xs.type() == precision)
            continue;
        const auto& calibrated = quant_params.at(any_cast<op::capture>(marker->get_operator()).ins_index);
        auto shift  = m.add_literal(literal{shape{precision}, std::vector<float>{calibrated.second}});
        auto scale  = m.add_literal(literal{shape{xs.type()}, std::vector<float>{qdq_scale_for(calibrated.first, xs.type())}});
        const auto over_x = make_op("multibroadcast", {{"out_lens", xs.lens()}});
        auto scales = m.insert_instruction(marker, over_x, scale);
        auto shifts = m.insert_instruction(marker, over_x, shift);
        auto stored = m.insert_instruction(marker, make_op("quantizelinear"), x, scales, shifts);
        m.replace_instruction(marker, make_op("dequantizelinear"), stored, scales, shifts);
    }
}

namespace {

// Calibration state of one quantization run: the largest magnitude every captured tensor has
// shown so far and the (multiplier, shift) pair that follows from it.  The multiplier maps the
// observed range onto the quantized type's, the shift stays 0 (quantization.cpp:88-130).
class range_calibration
{
    public:
    explicit range_calibration(shape::type_t precision)
    {
        switch(precision)
        {
        case shape::int8_type: target_range = 127.0f; break;
        case shape::fp8e4m3fnuz_type: target_range = 240.0f; break;
        case shape::fp8e4m3fn_type: target_range = 448.0f; break;
        default: MIGRAPHX_THROW("quantize: no 8-bit range for this type");
        }
    }

    void resize(std::size_t n)
    {
        largest.assign(n, 0.0f);
        parameters.assign(n, {64.0f, 0.0f}); // what a tensor that is never observed keeps
    }

    void observe(std::size_t index, const std::vector<float>& values)
    {
        float seen = largest.at(index);
        for(float v : values)
            seen = std::max(seen, std::fabs(v));
        largest.at(index)    = seen;
        parameters.at(index) = {seen == 0.0f ? 1.0f : target_range / seen, 0.0f};
    }

    std::vector<std::pair<float, float>> parameters;

    private:
    float target_range = 0.0f;
    std::vector<float> largest;
};

// quantization.cpp:132-174: mark the inputs of the named operators, run the marked program on
// the calibration data (on whatever target the caller chose, this build's included), then turn
// the marks into Q/DQ pairs
void calibrate_and_insert_qdq(program& prog,
                              const target& t,
                              shape::type_t precision,
                              const std::vector<parameter_map>& calibration,
                              const std::unordered_set<std::string>& ins_names)
{
    auto state = std::make_shared<range_calibration>(precision);
    auto on_capture = [state, t](std::size_t index, std::vector<argument> args) {
        state->observe(index, t.copy_from(args.front()).to_vector<float>());
    };
    std::size_t marked = 0;
    run_passes(prog, {capture_arguments_pass{ins_names, on_capture, &marked}});
    state->resize(marked);

    program marked_prog = prog;
    marked_prog.compile(t);
    for(const auto& sample : calibration)
    {
        parameter_map inputs;
        for(const auto& [name, param_shape] : marked_prog.get_parameter_shapes())
        {
            const auto given = sample.find(name);
            inputs[name]     = given != sample.end() ? t.copy_to(given->second) : t.allocate(param_shape);
        }
        marked_prog.eval(inputs);
        marked_prog.finish();
    }
    run_passes(prog, {quantize_8bits_pass{precision, state->parameters}, dead_code_elimination{}});
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
    calibrate_and_insert_qdq(prog, t, shape::int8_type, calibration, ins_names);
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
    calibrate_and_insert_qdq(prog, t, shape::fp8e4m3fn_type, calibration, names);
}

// ---------------------------------------------------------------- quantize int4

namespace {

// Per-tensor affine 4-bit parameters: the value range, widened to contain 0, mapped onto 0..15
// (quantize_int4.cpp:73-78)
struct uint4_affine
{
    float scale;
    int zero_point;

    static uint4_affine covering(const std::vector<float>& values)
    {
        const auto [lo_it, hi_it] = std::minmax_element(values.begin(), values.end());
        const float lo            = std::min(*lo_it, 0.0f);
        const float hi            = std::max(*hi_it, 0.0f);
        uint4_affine r{(hi - lo) / 15, 0};
        if(r.scale != 0)
            r.zero_point = static_cast<int>(std::round(-lo / r.scale));
        return r;
    }
};

// a constant float / half operand whose last axis can be packed two to a byte
bool can_store_as_int4(instruction_ref x)
{
    const auto& s = x->get_shape();
    if(s.broadcasted() or (s.type() != shape::float_type and s.type() != shape::half_type))
        return false;
    return s.lens().back() % 2 == 0 and x->can_eval();
}

// x -> dequantizelinear(unpack_int4(pack_int4(quantizelinear(x)))), all in front of `user`; the
// scale literals take the user's result type (quantize_int4.cpp:80-100)
instruction_ref through_int4(module& m, instruction_ref user, instruction_ref x)
{
    const auto values = x->eval().to_vector<float>();
    if(values.empty())
        return x;
    const auto affine = uint4_affine::covering(values);
    const auto over_x = make_op("multibroadcast", {{"out_lens", x->get_shape().lens()}});
    // the quantizing and the dequantizing side get literals of their own, as the reference's do
    auto parameters = [&] {
        auto s = m.add_literal(literal{shape{user->get_shape().type()}, std::vector<float>{affine.scale}});
        s      = m.insert_instruction(user, over_x, s);
        auto z = m.add_literal(literal{shape{shape::uint8_type}, std::vector<int>{affine.zero_point}});
        z      = m.insert_instruction(user, over_x, z);
        return std::make_pair(s, z);
    };
    const auto [qs, qz] = parameters();
    auto stored   = m.insert_instruction(user, make_op("quantizelinear"), x, qs, qz);
    auto packed   = m.insert_instruction(user, make_op("pack_int4", {{"axis", -1}}), stored);
    auto unpacked = m.insert_instruction(user, make_op("unpack_int4", {{"axis", -1}}), packed);
    const auto [ds, dz] = parameters();
    return m.insert_instruction(user, make_op("dequantizelinear"), unpacked, ds, dz);
}

} // namespace

// quantize_int4.cpp:38-103: constant float / half operands of dot and convolution go through a
// 4-bit store
void quantize_int4_pass::apply(module& m) const
{
    for(auto user : all_instructions(m))
    {
        if((user->name() != "dot" and user->name() != "convolution") or user->inputs().empty())
            continue;
        auto operands = user->inputs();
        for(auto& x : operands)
        {
            if(can_store_as_int4(x))
                x = through_int4(m, user, x);
        }
        if(operands != user->inputs())
            m.replace_instruction(user, user->get_operator(), operands);
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
