#include <cstdlib>
#include "device_ops.hpp"
#include <migraphx/ops.hpp>
#include <migraphx/passes.hpp>
#include <migraphx/register_op.hpp>
#include <algorithm>
#include <set>
#include <unordered_map>
#include <unordered_set>

namespace migraphx {
namespace mi355 {

namespace {

std::vector<instruction_ref> all_instructions(const module& m)
{
    std::vector<instruction_ref> r;
    for(auto it = m.begin(); it != m.end(); ++it)
        r.push_back(it);
    return r;
}

instruction_ref skip_broadcasts(instruction_ref i)
{
    while(i->name() == "broadcast" or i->name() == "multibroadcast")
        i = i->inputs().front();
    return i;
}

instruction_ref insert_allocation(module& m, instruction_ref ins, const shape& s)
{
    allocate a;
    a.s = s;
    return m.insert_instruction(ins, operation{a});
}

// a dense copy of `x` placed before `ins` when x is not in standard layout
instruction_ref make_standard(module& m, instruction_ref ins, instruction_ref x)
{
    if(x->get_shape().standard())
        return x;
    auto out = insert_allocation(m, ins, shape{x->get_shape().type(), x->get_shape().lens()});
    return m.insert_instruction(ins, operation{contiguous{}}, x, out);
}

// a quantization parameter the pointwise kernels can address with (row, column) strides
instruction_ref make_param(module& m, instruction_ref ins, instruction_ref p)
{
    int64_t sr = 0;
    int64_t sc = 0;
    if(collapse_2d(p->get_shape(), sr, sc))
        return p;
    auto out = insert_allocation(m, ins, shape{p->get_shape().type(), p->get_shape().lens()});
    return m.insert_instruction(ins, operation{contiguous{}}, p, out);
}

// value of a constant whose elements all are the same behind its broadcasts
bool scalar_constant(instruction_ref i, int64_t& v)
{
    auto base = skip_broadcasts(i);
    if(not base->can_eval() or base->get_shape().elements() == 0)
        return false;
    auto vals = base->eval().to_vector<int64_t>();
    if(not std::all_of(vals.begin(), vals.end(), [&](int64_t x) { return x == vals.front(); }))
        return false;
    v = vals.front();
    return true;
}

bool all_zero_constant(instruction_ref i)
{
    auto base = skip_broadcasts(i);
    if(not base->can_eval())
        return false;
    auto v = base->eval().to_vector<double>();
    return std::all_of(v.begin(), v.end(), [](double x) { return x == 0; });
}

// ---- quant_dot -> dequantizelinear [-> convert] --------------------------------------------

// the zero-point expression simplify_qdq builds (src/simplify_qdq.cpp:250-279):
//   0 [+ quant_dot(zp_a, B)] [+ quant_dot(A, zp_b)] [- quant_dot(zp_a, zp_b)]
struct zp_terms
{
    bool ok      = true;
    int64_t zp_a = 0;
    int64_t zp_b = 0;
    bool seen_a = false, seen_b = false, seen_ab = false;
};

void parse_zp(instruction_ref e, instruction_ref a, instruction_ref b, bool negated, zp_terms& t)
{
    if(not t.ok)
        return;
    if(e->name() == "add")
    {
        parse_zp(e->inputs()[0], a, b, negated, t);
        parse_zp(e->inputs()[1], a, b, negated, t);
        return;
    }
    if(e->name() == "sub")
    {
        parse_zp(e->inputs()[0], a, b, negated, t);
        parse_zp(e->inputs()[1], a, b, not negated, t);
        return;
    }
    if(e->name() == "multibroadcast" or e->name() == "broadcast" or e->name() == "@literal")
    {
        t.ok = t.ok and not negated and all_zero_constant(e);
        return;
    }
    if(e->name() != "quant_dot" or e->inputs().size() != 2)
    {
        t.ok = false;
        return;
    }
    auto l = e->inputs()[0];
    auto r = e->inputs()[1];
    int64_t vl = 0;
    int64_t vr = 0;
    const bool cl = l != a and scalar_constant(l, vl);
    const bool cr = r != b and scalar_constant(r, vr);
    if(cl and r == b and not negated and not t.seen_a)
    {
        t.zp_a   = vl;
        t.seen_a = true;
    }
    else if(l == a and cr and not negated and not t.seen_b)
    {
        t.zp_b   = vr;
        t.seen_b = true;
    }
    else if(cl and cr and negated and not t.seen_ab)
    {
        t.seen_ab = true;
        // checked against the two single terms once all are known
        if((t.seen_a and t.zp_a != vl) or (t.seen_b and t.zp_b != vr))
            t.ok = false;
        t.zp_a = vl;
        t.zp_b = vr;
    }
    else
    {
        t.ok = false;
    }
}

// how a scale broadcast to the [.., M, N] result varies: per tensor, per row or per column
int scale_mode(const shape& s)
{
    const std::size_t nd = s.ndim();
    bool row = false;
    bool col = false;
    for(std::size_t i = 0; i < nd; i++)
    {
        if(s.lens()[i] == 1 or s.strides()[i] == 0)
            continue;
        if(i == nd - 2 and s.strides()[i] == 1)
            row = true;
        else if(i == nd - 1 and s.strides()[i] == 1)
            col = true;
        else
            return -1;
    }
    if(row and col)
        return -1;
    return row ? MI355_QP_PER_ROW : (col ? MI355_QP_PER_COL : MI355_QP_PER_TENSOR);
}

// a float [N] vector broadcast over every row of `lens`
bool is_column_bias(instruction_ref x, const std::vector<std::size_t>& lens)
{
    const shape& s = x->get_shape();
    if(s.type() != shape::float_type or s.lens() != lens)
        return false;
    const std::size_t nd = s.ndim();
    for(std::size_t i = 0; i + 1 < nd; i++)
    {
        if(s.lens()[i] != 1 and s.strides()[i] != 0)
            return false;
    }
    if(s.lens()[nd - 1] != 1 and s.strides()[nd - 1] != 1)
        return false;
    auto base = skip_broadcasts(x);
    return base != x and base->get_shape().type() == shape::float_type and base->get_shape().standard() and
           base->get_shape().elements() == lens.back();
}

// A skinny int8 product splits K over the chip when it is given room for the partial sums: ask
// the library how much this shape can use and pass it as one more buffer.
void add_dot_workspace(module& m, instruction_ref pos, quant_dot& op, std::vector<instruction_ref>& args)
{
    const auto d      = op.describe(args[0]->get_shape(), args[1]->get_shape());
    const size_t need = mi355_quant_dot_workspace_size(&d);
    if(need == 0)
        return;
    op.workspace = true;
    args.push_back(insert_allocation(m, pos, shape{shape::uint8_type, {need}}));
}

bool fuse_quant_dot_dq(module& m, instruction_ref dq)
{
    if(dq->name() != "dequantizelinear")
        return false;
    auto qd = dq->inputs()[0];
    if(qd->name() != "quant_dot" or qd->inputs().size() != 2 or qd->outputs().size() != 1)
        return false;
    auto a = qd->inputs()[0];
    auto b = qd->inputs()[1];
    if(not view_as_matrix(a->get_shape()).ok or not view_as_matrix(b->get_shape()).ok)
        return false;
    auto scale = dq->inputs()[1];
    if(scale->get_shape().type() != shape::float_type)
        return false;

    // scale: mul(bcast(s1), bcast(s2)) or one broadcast tensor
    instruction_ref sa = scale;
    instruction_ref sb = scale;
    int mode_a         = MI355_QP_NONE;
    int mode_b         = MI355_QP_NONE;
    if(scale->name() == "mul")
    {
        sa     = scale->inputs()[0];
        sb     = scale->inputs()[1];
        mode_a = scale_mode(sa->get_shape());
        mode_b = scale_mode(sb->get_shape());
        if(mode_a == MI355_QP_PER_COL and mode_b != MI355_QP_PER_COL)
        {
            std::swap(sa, sb);
            std::swap(mode_a, mode_b);
        }
        else if(mode_b == MI355_QP_PER_ROW and mode_a != MI355_QP_PER_ROW)
        {
            std::swap(sa, sb);
            std::swap(mode_a, mode_b);
        }
        if(mode_a < 0 or mode_b < 0 or mode_a == MI355_QP_PER_COL or mode_b == MI355_QP_PER_ROW)
            return false;
    }
    else
    {
        const int mode = scale_mode(scale->get_shape());
        if(mode < 0)
            return false;
        if(mode == MI355_QP_PER_COL)
            mode_b = mode;
        else
            mode_a = mode;
    }

    zp_terms t;
    if(dq->inputs().size() == 3)
    {
        parse_zp(dq->inputs()[2], a, b, false, t);
        if(not t.ok)
            return false;
        // both zero points set needs the cross term, one alone must not have it
        if(t.seen_ab != (t.seen_a and t.seen_b))
            return false;
        if(not t.seen_a)
            t.zp_a = 0;
        if(not t.seen_b)
            t.zp_b = 0;
        if((t.zp_a != 0 or t.zp_b != 0) and
           (a->get_shape().type() != shape::int8_type or view_as_matrix(a->get_shape()).batch != 1))
            return false;
    }

    // an only user that converts to a 16-bit float joins the epilogue
    instruction_ref last   = dq;
    shape::type_t out_type = shape::float_type;
    if(dq->outputs().size() == 1 and dq->outputs().front()->name() == "convert")
    {
        auto cv = dq->outputs().front();
        auto tt = any_cast<op::convert>(cv->get_operator()).target_type;
        if(tt == shape::half_type or tt == shape::bf16_type)
        {
            last     = cv;
            out_type = tt;
        }
    }

    // so does the bias of a linear layer: an only user that adds a vector broadcast along the rows
    // (the epilogue adds it in fp32 exactly as the `add` would)
    bool has_bias = false;
    instruction_ref bias;
    if(last == dq and dq->outputs().size() == 1 and dq->outputs().front()->name() == "add")
    {
        auto add   = dq->outputs().front();
        auto other = add->inputs()[0] == dq ? add->inputs()[1] : add->inputs()[0];
        if(other != dq and is_column_bias(other, qd->get_shape().lens()))
        {
            has_bias = true;
            bias     = skip_broadcasts(other);
            last     = add;
        }
    }

    quant_dot op;
    op.dequant      = true;
    op.has_bias     = has_bias;
    op.zp_a         = t.zp_a;
    op.zp_b         = t.zp_b;
    op.scale_a_mode = mode_a;
    op.scale_b_mode = mode_b;
    op.out_type     = out_type;
    // an absent scale still needs a pointer-sized argument: pass the other one, its mode is NONE
    std::vector<instruction_ref> args = {a, b, sa, sb};
    if(t.zp_a != 0)
    {
        const auto n = b->get_shape().lens().back();
        auto buf     = insert_allocation(m, last, shape{shape::int32_type, {n}});
        args.push_back(m.insert_instruction(last, operation{colsum{}}, b, buf));
    }
    if(t.zp_b != 0)
    {
        const auto rows = a->get_shape().lens()[a->get_shape().ndim() - 2];
        auto buf        = insert_allocation(m, last, shape{shape::int32_type, {rows}});
        args.push_back(m.insert_instruction(last, operation{rowsum{}}, a, buf));
    }
    if(has_bias)
        args.push_back(bias);
    add_dot_workspace(m, last, op, args);
    args.push_back(insert_allocation(m, last, shape{out_type, qd->get_shape().lens()}));
    m.replace_instruction(last, operation{op}, args);
    return true;
}

// ---- quant_convolution [-> dequantizelinear [-> convert]] --------------------------------------

quant_convolution conv_operator(instruction_ref qc)
{
    const auto& ref = any_cast<op::quant_convolution>(qc->get_operator());
    quant_convolution op;
    op.padding  = ref.padding;
    op.stride   = ref.stride;
    op.dilation = ref.dilation;
    op.group    = ref.group;
    op.out_type = qc->get_shape().type();
    return op;
}

instruction_ref insert_conv_workspace(module& m, instruction_ref pos, const quant_convolution& op,
                                      instruction_ref x, instruction_ref w)
{
    const auto d = op.describe(x->get_shape(), w->get_shape());
    size_t need  = 0;
    if(mi355_quant_convolution3d_dims(&d, nullptr, &need) != MI355_OK)
        MIGRAPHX_THROW("mi355: quant_convolution attributes are not valid");
    return insert_allocation(m, pos, shape{shape::uint8_type, {std::max<std::size_t>(need, 16)}});
}

// 0: one value, 1: one value per channel (axis 1) of `lens`, -1: anything else
int channel_scale_mode(instruction_ref x, const std::vector<std::size_t>& lens)
{
    const shape& s = x->get_shape();
    if(s.type() != shape::float_type or s.lens() != lens)
        return -1;
    auto base = skip_broadcasts(x);
    if(not base->get_shape().standard())
        return -1;
    bool channel = false;
    for(std::size_t i = 0; i < s.ndim(); i++)
    {
        if(s.lens()[i] == 1 or s.strides()[i] == 0)
            continue;
        if(i == 1 and s.strides()[i] == 1)
            channel = true;
        else
            return -1;
    }
    if(channel)
        return base->get_shape().elements() == lens[1] ? 1 : -1;
    return base->get_shape().elements() == 1 ? 0 : -1;
}

// What simplify_qdq leaves of a convolution with symmetric zero points (simplify_qdq.cpp:171-222
// after remove_zero_point): quant_convolution -> dequantizelinear(., mul(bcast(scale_x),
// bcast(scale_w))) [-> convert to a 16-bit float].  One operator: the GEMM's epilogue scales.
bool fuse_quant_conv_dq(module& m, instruction_ref dq)
{
    if(dq->name() != "dequantizelinear" or dq->inputs().size() != 2)
        return false;
    auto qc = dq->inputs()[0];
    if(qc->name() != "quant_convolution" or qc->inputs().size() != 2 or qc->outputs().size() != 1)
        return false;
    auto scale = dq->inputs()[1];
    if(scale->name() != "mul" or scale->get_shape().type() != shape::float_type)
        return false;
    const auto& lens = qc->get_shape().lens();
    auto s1          = scale->inputs()[0];
    auto s2          = scale->inputs()[1];
    int m1           = channel_scale_mode(s1, lens);
    int m2           = channel_scale_mode(s2, lens);
    if(m1 == 1 and m2 == 0)
    {
        std::swap(s1, s2);
        std::swap(m1, m2);
    }
    if(m1 != 0 or m2 < 0)
        return false;
    const auto t = qc->inputs()[0]->get_shape().type();
    if(t != shape::int8_type and t != shape::fp8e4m3fn_type)
        return false;
    const std::size_t kd = qc->get_shape().ndim() - 2;
    if(kd < 1 or kd > 3)
        return false;

    instruction_ref last   = dq;
    shape::type_t out_type = shape::float_type;
    if(dq->outputs().size() == 1 and dq->outputs().front()->name() == "convert")
    {
        auto cv = dq->outputs().front();
        auto tt = any_cast<op::convert>(cv->get_operator()).target_type;
        if(tt == shape::half_type or tt == shape::bf16_type)
        {
            last     = cv;
            out_type = tt;
        }
    }
    auto op         = conv_operator(qc);
    op.dequant      = true;
    op.scale_w_mode = m2 == 1 ? MI355_QP_PER_ROW : MI355_QP_PER_TENSOR;
    op.out_type     = out_type;
    auto x          = make_standard(m, last, qc->inputs()[0]);
    auto w          = make_standard(m, last, qc->inputs()[1]);
    auto ws         = insert_conv_workspace(m, last, op, x, w);
    auto out        = insert_allocation(m, last, shape{out_type, lens});
    m.replace_instruction(last, operation{op}, {x, w, skip_broadcasts(s1), skip_broadcasts(s2), ws, out});
    return true;
}

// ---- dot(x, transpose(dequantizelinear(unpack_int4(w), blockwise scales, zero points))) -------

instruction_ref skip_full_slice(instruction_ref x, bool& sliced)
{
    sliced = false;
    if(x->name() == "slice")
    {
        sliced = true;
        return x->inputs().front();
    }
    return x;
}

// x = reshape{n,-1}(multibroadcast{[n, nblk, blk]}(unsqueeze{2}(base [n, nblk]))): every element
// of base repeated blk times along the last axis (src/onnx/parse_matmulnbits.cpp:140-158)
bool match_blockwise(instruction_ref x, std::size_t n, instruction_ref& base, std::size_t& blk)
{
    bool sliced = false;
    x           = skip_full_slice(x, sliced);
    if(sliced)
        return false; // a runt block: K is not a multiple of the block size
    if(x->name() != "reshape")
        return false;
    auto mb = x->inputs().front();
    if(mb->name() != "multibroadcast" or mb->get_shape().ndim() != 3 or mb->get_shape().lens()[0] != n)
        return false;
    auto us = mb->inputs().front();
    if(us->name() != "unsqueeze" or us->get_shape().ndim() != 3 or us->get_shape().lens()[2] != 1)
        return false;
    base = us->inputs().front();
    if(base->get_shape().ndim() != 2 or not base->get_shape().standard())
        return false;
    blk = mb->get_shape().lens()[2];
    return true;
}

bool unpacks_last_axis(instruction_ref unpk)
{
    const auto axis = any_cast<op::unpack_int4>(unpk->get_operator()).axis;
    return axis == -1 or axis == static_cast<int64_t>(unpk->get_shape().ndim()) - 1;
}

bool lower_w4a16(module& m, instruction_ref ins)
{
    auto a  = ins->inputs()[0];
    auto bt = ins->inputs()[1];
    if(a->get_shape().type() != shape::half_type or a->get_shape().ndim() != 2)
        return false;
    if(bt->name() != "transpose")
        return false;
    auto dq = bt->inputs().front();
    if(dq->name() != "dequantizelinear" or dq->get_shape().ndim() != 2 or
       dq->get_shape().type() != shape::half_type)
        return false;
    const auto n = dq->get_shape().lens()[0];
    const auto k = dq->get_shape().lens()[1];
    bool sliced  = false;
    auto unpk    = skip_full_slice(dq->inputs()[0], sliced);
    if(sliced or unpk->name() != "unpack_int4" or unpk->get_shape().type() != shape::uint8_type)
        return false;
    auto packed = unpk->inputs().front();
    if(not packed->get_shape().standard() or packed->get_shape().ndim() != 2)
        return false;
    // the kernel reads nibble pairs along K: the unpack must run along the last axis of [N, K/2]
    // (a weight packed along axis 0 has the same byte count and would be read the wrong way)
    if(not unpacks_last_axis(unpk) or packed->get_shape().lens() != std::vector<std::size_t>{n, k / 2} or k % 2 != 0)
        return false;

    instruction_ref scales;
    std::size_t blk = 0;
    if(not match_blockwise(dq->inputs()[1], n, scales, blk))
        return false;
    if(blk % 32 != 0 or k % blk != 0 or scales->get_shape().lens()[1] != k / blk)
        return false;

    w4a16_gemm op;
    op.group = static_cast<int64_t>(blk);
    std::vector<instruction_ref> args = {a, packed, scales};
    if(dq->inputs().size() == 2)
    {
        op.zp_mode   = MI355_W4_ZP_SCALAR;
        op.zp_scalar = 0;
    }
    else
    {
        auto z    = dq->inputs()[2];
        int64_t v = 0;
        instruction_ref zbase;
        std::size_t zblk = 0;
        if(scalar_constant(z, v))
        {
            if(v < 0 or v > 15)
                return false; // not a 4-bit zero point: the generic operators take the graph
            op.zp_mode   = MI355_W4_ZP_SCALAR;
            op.zp_scalar = v;
        }
        else if(match_blockwise(z, n, zbase, zblk) and zblk == blk)
        {
            bool zsliced = false;
            auto zu      = skip_full_slice(zbase, zsliced);
            if(zu->name() == "unpack_int4" and zu->inputs().front()->get_shape().standard() and
               unpacks_last_axis(zu) and zu->inputs().front()->get_shape().ndim() == 2 and
               zu->inputs().front()->get_shape().lens()[0] == n)
            {
                op.zp_mode = MI355_W4_ZP_PACKED;
                args.push_back(zu->inputs().front());
            }
            else if(not zsliced and zbase->get_shape().type() == shape::uint8_type)
            {
                op.zp_mode = MI355_W4_ZP_GROUP;
                args.push_back(zbase);
            }
            else
                return false;
        }
        else
            return false;
    }
    // the kernels load 16 bytes of a row at a time: rows must start 16-byte aligned
    if((a->get_shape().strides()[1] != 1 and a->get_shape().lens()[1] != 1) or
       a->get_shape().strides()[0] % 8 != 0 or a->name() == "slice")
        args[0] = make_standard(m, ins, a);
    // room for split-K partial sums where the column tiles alone do not fill the chip
    const auto rows   = a->get_shape().lens()[0];
    const size_t need = mi355_w4a16_gemm_workspace_size(static_cast<int64_t>(rows), static_cast<int64_t>(n),
                                                        static_cast<int64_t>(k), op.group);
    if(need > 0)
    {
        op.workspace = true;
        args.push_back(insert_allocation(m, ins, shape{shape::uint8_type, {need}}));
    }
    args.push_back(insert_allocation(m, ins, shape{shape::half_type, {rows, n}}));
    m.replace_instruction(ins, operation{op}, args);
    return true;
}

// ---- weight-only GEMMs that share their activations -> one launch -------------------------------
//
// The q / k / v projections of an attention layer and the gate / up projections of its MLP multiply
// the same activations by different constant weights.  At one row of activations such a product
// is a few microseconds of weight streaming behind a launch and a fetch of the activations that
// cost as much; with the weights (and their scales) stacked along N at compile time the products
// become one launch, and each original result is a `slice` of its columns.  A column's sum does
// not depend on which other columns are computed with it (the reordered one-row form splits K over
// more or fewer waves with the number of columns, which can move a sum's last bit between a very
// wide and a narrow product; the tolerance of the path covers it).
// Taken: scalar zero points, weights and scales known at compile time, the same activations,
// K, group size and zero point.
void fuse_shared_w4a16(module& m)
{
    std::vector<instruction_ref> gemms;
    for(auto ins : all_instructions(m))
    {
        if(ins->name() == "mi355::w4a16_gemm")
            gemms.push_back(ins);
    }
    auto constant = [](instruction_ref x) { return x->can_eval() and x->get_shape().standard(); };
    std::unordered_set<const instruction*> taken;
    for(std::size_t i = 0; i < gemms.size(); i++)
    {
        auto first = gemms[i];
        if(taken.count(&*first) > 0)
            continue;
        const auto op = any_cast<w4a16_gemm>(first->get_operator());
        if(op.zp_mode != MI355_W4_ZP_SCALAR or not constant(first->inputs()[1]) or not constant(first->inputs()[2]))
            continue;
        const auto k2 = first->inputs()[1]->get_shape().lens()[1];
        const auto kb = first->inputs()[2]->get_shape().lens()[1];
        std::vector<instruction_ref> members = {first};
        for(std::size_t j = i + 1; j < gemms.size(); j++)
        {
            auto other = gemms[j];
            if(taken.count(&*other) > 0 or other->inputs()[0] != first->inputs()[0])
                continue;
            const auto oop = any_cast<w4a16_gemm>(other->get_operator());
            if(oop.zp_mode != MI355_W4_ZP_SCALAR or oop.zp_scalar != op.zp_scalar or oop.group != op.group or
               not constant(other->inputs()[1]) or not constant(other->inputs()[2]) or
               other->inputs()[1]->get_shape().lens()[1] != k2 or other->inputs()[2]->get_shape().lens()[1] != kb or
               other->inputs()[2]->get_shape().type() != first->inputs()[2]->get_shape().type())
                continue;
            members.push_back(other);
        }
        // Each member's result becomes a column slice of the stacked one, a view whose rows start
        // at the member's first column: a kernel that takes such a view as its activations reads 16
        // bytes at a time, so every member's column count must keep the slices 16-byte aligned.
        members.erase(std::remove_if(members.begin() + 1,
                                     members.end(),
                                     [](instruction_ref g) { return g->inputs()[1]->get_shape().lens()[0] % 8 != 0; }),
                      members.end());
        if(members.size() < 2 or first->inputs()[1]->get_shape().lens()[0] % 8 != 0)
            continue;
        std::size_t n = 0;
        std::string weights, scales;
        for(auto g : members)
        {
            taken.insert(&*g);
            const argument w = g->inputs()[1]->eval();
            const argument s = g->inputs()[2]->eval();
            weights.append(w.data(), w.get_shape().bytes());
            scales.append(s.data(), s.get_shape().bytes());
            n += g->inputs()[1]->get_shape().lens()[0];
        }
        auto a          = first->inputs()[0];
        const auto rows = a->get_shape().lens()[0];
        auto wl = m.add_literal(literal{shape{shape::uint8_type, {n, k2}}, weights.data()});
        auto sl = m.add_literal(literal{shape{first->inputs()[2]->get_shape().type(), {n, kb}}, scales.data()});
        w4a16_gemm fused = op;
        fused.workspace  = false;
        std::vector<instruction_ref> args = {a, wl, sl};
        const size_t need = mi355_w4a16_gemm_workspace_size(static_cast<int64_t>(rows), static_cast<int64_t>(n),
                                                            static_cast<int64_t>(2 * k2), op.group);
        if(need > 0)
        {
            fused.workspace = true;
            args.push_back(insert_allocation(m, first, shape{shape::uint8_type, {need}}));
        }
        args.push_back(insert_allocation(m, first, shape{shape::half_type, {rows, n}}));
        auto all = m.insert_instruction(first, operation{fused}, args);
        std::size_t at = 0;
        for(auto g : members)
        {
            const auto cols = g->inputs()[1]->get_shape().lens()[0];
            m.replace_instruction(g,
                                  make_op("slice", {{"axes", {1}},
                                                    {"starts", {static_cast<int64_t>(at)}},
                                                    {"ends", {static_cast<int64_t>(at + cols)}}}),
                                  {all});
            at += cols;
        }
    }
}

// ---- quantized layers that share their activations -> one batched launch ----------------------
//
// The q / k / v projections of an attention block are three mi355::quant_dot over the same int8
// activations with constant weights of one shape.  At 12288 x 768 x 768 each is 144 output tiles on
// a chip of 256 CUs: a launch that leaves CUs idle and lasts one tile's pipeline fill, 12 K slabs and
// a 256 KB store.  Stacked along a batch axis at compile time -- the activations broadcast with a
// batch stride of 0, the weights [3, K, N], the column scales and the biases [3, N]
// (MI355_QP_PER_COL_BATCH) -- they are one launch of 432 tiles, and each layer's result is one
// dense [M, N] block of the stacked result, so nothing downstream changes.  The sums are the same
// integers and the epilogue the same operations: the same bits.
// Taken: dequantizing int8 products without zero points, one scale for the activations (the same
// instruction), per-column weight scales, weights / scales / biases known at compile time and
// dense, at least 128 rows, fewer tiles than CUs in one member's launch.
// MIGRAPHX_MI355_DISABLE_SHARED_QUANT_DOT set (to anything but 0) when a program is compiled keeps
// the launches separate.
void fuse_shared_quant_dots(module& m)
{
    const char* off = std::getenv("MIGRAPHX_MI355_DISABLE_SHARED_QUANT_DOT");
    if(off != nullptr and std::string(off) != "0")
        return;
    std::vector<instruction_ref> gemms;
    for(auto ins : all_instructions(m))
    {
        if(ins->name() == "mi355::quant_dot")
            gemms.push_back(ins);
    }
    auto constant = [](instruction_ref x) { return x->can_eval() and x->get_shape().standard(); };
    // a, b, scale_a, scale_b, [bias], out
    auto candidate = [&](instruction_ref g, const quant_dot& op) {
        if(not op.dequant or op.zp_a != 0 or op.zp_b != 0 or op.workspace or
           op.scale_a_mode != MI355_QP_PER_TENSOR or op.scale_b_mode != MI355_QP_PER_COL)
            return false;
        const shape& a = g->inputs()[0]->get_shape();
        const shape& b = g->inputs()[1]->get_shape();
        // the column scales arrive as a [N] constant broadcast over the rows
        if(a.type() != shape::int8_type or a.ndim() != 2 or not a.standard() or b.ndim() != 2 or
           not constant(g->inputs()[1]) or not constant(skip_broadcasts(g->inputs()[3])) or
           (op.has_bias and not constant(g->inputs()[4])))
            return false;
        const auto rows = a.lens()[0], k = a.lens()[1], n = b.lens()[1];
        const auto tiles = ((rows + 255) / 256) * ((n + 255) / 256);
        return rows >= 128 and k % 64 == 0 and n % 16 == 0 and tiles < 256 and
               skip_broadcasts(g->inputs()[3])->get_shape().elements() == n;
    };
    std::unordered_set<const instruction*> taken;
    for(std::size_t i = 0; i < gemms.size(); i++)
    {
        auto first = gemms[i];
        if(taken.count(&*first) > 0)
            continue;
        const auto op = any_cast<quant_dot>(first->get_operator());
        if(not candidate(first, op))
            continue;
        std::vector<instruction_ref> members = {first};
        for(std::size_t j = i + 1; j < gemms.size(); j++)
        {
            auto other = gemms[j];
            if(taken.count(&*other) > 0 or &*other->inputs()[0] != &*first->inputs()[0] or
               &*skip_broadcasts(other->inputs()[2]) != &*skip_broadcasts(first->inputs()[2]))
                continue;
            const auto oop = any_cast<quant_dot>(other->get_operator());
            if(not candidate(other, oop) or oop.has_bias != op.has_bias or oop.out_type != op.out_type or
               other->inputs()[1]->get_shape() != first->inputs()[1]->get_shape())
                continue;
            members.push_back(other);
        }
        if(members.size() < 2)
            continue;
        // the stacked launch goes where the first member is: every member's operands are defined
        // there already (the shared ones are the first member's, the others are constants, which
        // become literals of their own below)
        std::string weights, scales, biases;
        for(auto g : members)
        {
            taken.insert(&*g);
            const argument w = g->inputs()[1]->eval();
            const argument sc = skip_broadcasts(g->inputs()[3])->eval();
            weights.append(w.data(), w.get_shape().bytes());
            scales.append(sc.data(), sc.get_shape().bytes());
            if(op.has_bias)
            {
                const argument bi = g->inputs()[4]->eval();
                biases.append(bi.data(), bi.get_shape().bytes());
            }
        }
        auto a           = first->inputs()[0];
        const auto nb    = members.size();
        const auto rows  = a->get_shape().lens()[0];
        const auto k     = a->get_shape().lens()[1];
        const auto n     = first->inputs()[1]->get_shape().lens()[1];
        auto ab = m.insert_instruction(first, make_op("multibroadcast", {{"out_lens", {nb, rows, k}}}), a);
        auto wl = m.add_literal(literal{shape{shape::int8_type, {nb, k, n}}, weights.data()});
        auto sl = m.add_literal(literal{shape{shape::float_type, {nb, n}}, scales.data()});
        quant_dot fused    = op;
        fused.scale_b_mode = MI355_QP_PER_COL_BATCH;
        std::vector<instruction_ref> args = {ab, wl, first->inputs()[2], sl};
        if(op.has_bias)
            args.push_back(m.add_literal(literal{shape{shape::float_type, {nb, n}}, biases.data()}));
        args.push_back(insert_allocation(m, first, shape{op.out_type, {nb, rows, n}}));
        auto all = m.insert_instruction(first, operation{fused}, args);
        for(std::size_t at = 0; at < nb; at++)
        {
            auto one = m.insert_instruction(members[at],
                                            make_op("slice", {{"axes", {0}},
                                                              {"starts", {static_cast<int64_t>(at)}},
                                                              {"ends", {static_cast<int64_t>(at + 1)}}}),
                                            all);
            m.replace_instruction(members[at], make_op("squeeze", {{"axes", {0}}}), {one});
        }
    }
}

// ---- weight-only products of a few rows over constant weights -> the reordered form -------------
//
// With one row of activations (or a few: a small batch) the product is a stream of weights, and constant weights can lie in
// memory in whatever order the kernel reads fastest.  mi355::w4a16_prepack writes that order; its
// operands are literals, so it runs once when the program is compiled (constant folding, below)
// and the program keeps only the reordered copy.  Taken: one zero point for the tensor, group size
// 128, the shapes mi355_w4a16_prepacked_size accepts and at most mi355_w4a16_prepacked_max_rows rows
// (dense when more than one); everything else stays on mi355::w4a16_gemm.
void prepack_w4a16(module& m)
{
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "mi355::w4a16_gemm")
            continue;
        const auto op = any_cast<w4a16_gemm>(ins->get_operator());
        auto a        = ins->inputs()[0];
        auto w        = ins->inputs()[1];
        auto s        = ins->inputs()[2];
        if(op.zp_mode != MI355_W4_ZP_SCALAR or op.group != 128)
            continue;
        if(not(w->can_eval() and w->get_shape().standard() and s->can_eval() and s->get_shape().standard()))
            continue;
        const auto n       = static_cast<int64_t>(w->get_shape().lens()[0]);
        const auto k       = static_cast<int64_t>(w->get_shape().lens()[1] * 2);
        const size_t bytes = mi355_w4a16_prepacked_size(n, k, op.group);
        if(bytes == 0)
            continue;
        // one row always; a few rows (small batches) while they fit the LDS, rows 16-byte aligned
        const auto rows = static_cast<int64_t>(a->get_shape().lens()[0]);
        if(rows > mi355_w4a16_prepacked_max_rows(n, k, op.group))
            continue;
        if(rows > 1 and not a->get_shape().standard())
            continue;
        w4a16_prepack pre;
        pre.zp_scalar = op.zp_scalar;
        auto room     = insert_allocation(m, ins, shape{shape::uint8_type, {bytes}});
        auto packed   = m.insert_instruction(ins, operation{pre}, w, s, room);
        m.replace_instruction(ins, operation{w4a16_gemm_prepacked{}}, a, packed, ins->inputs().back());
    }
}

// ---- quant_dot of a few rows against a constant B -> the reordered form --------------------------
//
// A linear layer applied to at most 16 rows (decoding, small batches) is a stream of its weight
// matrix.  When B is built from literals only, mi355::quant_dot_prepack -- folded when the program
// is compiled, like the step above -- stores it as the matrix-core operand tiles, and
// mi355::quant_dot_prepacked computes the layer in one launch, without the split-K workspace and
// its second kernel.  Taken: one batch, A dense [M <= 16, K], the shapes
// mi355_quant_dot_prepacked_size accepts; everything else stays on mi355::quant_dot.
bool built_from_literals(instruction_ref ins, std::unordered_map<const instruction*, bool>& seen)
{
    auto it = seen.find(&*ins);
    if(it != seen.end())
        return it->second;
    bool r = false;
    if(ins->name() == "@literal" or ins->name() == "mi355::literal")
        r = true;
    else if(ins->name()[0] != '@' and ins->name() != "mi355::allocate" and not ins->inputs().empty())
    {
        r = true;
        for(auto i : ins->inputs())
        {
            if(i->name() == "mi355::allocate")
                continue;
            r = r and built_from_literals(i, seen);
        }
    }
    seen[&*ins] = r;
    return r;
}

// MIGRAPHX_MI355_DISABLE_PREPACK_QUANT_DOT set (to anything but 0) when a program is compiled keeps
// these layers on mi355::quant_dot with its split-K workspace.
bool prepack_quant_dot_enabled()
{
    const char* v = std::getenv("MIGRAPHX_MI355_DISABLE_PREPACK_QUANT_DOT");
    return v == nullptr or std::string(v) == "0" or std::string(v) == "";
}

void prepack_quant_dot(module& m)
{
    std::unordered_map<const instruction*, bool> seen;
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "mi355::quant_dot")
            continue;
        const auto op = any_cast<quant_dot>(ins->get_operator());
        auto inputs   = ins->inputs();
        auto a        = inputs[0];
        auto b        = inputs[1];
        const auto& as = a->get_shape();
        const auto& bs = b->get_shape();
        if(as.ndim() != 2 or bs.ndim() != 2 or not as.standard() or as.lens()[0] > 16)
            continue;
        if(as.type() == shape::uint8_type or not view_as_matrix(bs).ok)
            continue;
        const size_t bytes =
            mi355_quant_dot_prepacked_size(to_mi355_type(as.type()), bs.lens()[1], bs.lens()[0]);
        if(bytes == 0 or not built_from_literals(b, seen))
            continue;
        quant_dot_prepacked pre;
        pre.dequant      = op.dequant;
        pre.has_bias     = op.has_bias;
        pre.zp_a         = op.zp_a;
        pre.zp_b         = op.zp_b;
        pre.scale_a_mode = op.scale_a_mode;
        pre.scale_b_mode = op.scale_b_mode;
        pre.out_type     = op.out_type;
        auto room   = insert_allocation(m, ins, shape{shape::uint8_type, {bytes}});
        auto packed = m.insert_instruction(ins, operation{quant_dot_prepack{}}, b, room);
        std::vector<instruction_ref> args = inputs;
        args[1] = packed;
        if(op.workspace) // the buffer in front of the output
            args.erase(args.end() - 2);
        m.replace_instruction(ins, operation{pre}, args);
    }
}

// MIGRAPHX_MI355_FP32_DOT set (to anything but 0) when a program is compiled: float `dot`s run on
// the fp32 matrix cores instead of reproducing the reference's double sum bit for bit
bool fp32_dot_requested()
{
    const char* v = std::getenv("MIGRAPHX_MI355_FP32_DOT");
    return v != nullptr and std::string(v) != "0" and std::string(v) != "";
}

// ---- dot -> mul by one value (attention scores) -------------------------------------------------
// The multiplication joins the dot's store: float(sum) * value, the two roundings the two
// operators perform.
bool fuse_dot_scale(module& m, instruction_ref mul)
{
    if(mul->name() != "mul" or mul->get_shape().type() != shape::float_type)
        return false;
    for(int side = 0; side < 2; side++)
    {
        auto d = mul->inputs()[side];
        auto s = mul->inputs()[1 - side];
        if(d->name() != "dot" or d->outputs().size() != 1 or d->get_shape().type() != shape::float_type)
            continue;
        auto base = skip_broadcasts(s);
        if(base == s or base->get_shape().elements() != 1 or base->get_shape().type() != shape::float_type or
           s->get_shape().lens() != d->get_shape().lens())
            continue;
        auto a = d->inputs()[0];
        auto b = d->inputs()[1];
        if(not batch_collapses(a->get_shape()) and a->get_shape().ndim() != 4)
            a = make_standard(m, mul, a);
        if(not batch_collapses(b->get_shape()) and b->get_shape().ndim() != 4)
            b = make_standard(m, mul, b);
        dot op;
        op.scaled  = true;
        op.fp32acc = fp32_dot_requested();
        auto out   = insert_allocation(m, mul, shape{shape::float_type, d->get_shape().lens()});
        m.replace_instruction(mul, operation{op}, {a, b, base, out});
        return true;
    }
    return false;
}

// ---- chains of float pointwise operators ------------------------------------------------------
//
// add / sub / mul / div and the unary functions that feed one another through single-use values
// become one mi355::chain, which keeps the intermediate values in registers.  The reference
// groups such operators into pointwise modules (src/fuse_pointwise.cpp:364-385) and compiles
// each module; here the group is restricted to what a machine with the running value and one
// saved value can evaluate, which covers the encoder's GELU, bias + residual and the
// scale-and-shift tail of layer normalisation.  The steps repeat the operators in their own
// order, so the fused result equals the unfused one bit for bit.

int binary_code(const std::string& name)
{
    if(name == "add")
        return MI355_BIN_ADD;
    if(name == "sub")
        return MI355_BIN_SUB;
    if(name == "mul")
        return MI355_BIN_MUL;
    if(name == "div")
        return MI355_BIN_DIV;
    return -1;
}

int unary_code(const std::string& name)
{
    if(name == "erf")
        return MI355_UN_ERF;
    if(name == "sqrt")
        return MI355_UN_SQRT;
    if(name == "rsqrt")
        return MI355_UN_RSQRT;
    if(name == "exp")
        return MI355_UN_EXP;
    if(name == "tanh")
        return MI355_UN_TANH;
    if(name == "neg")
        return MI355_UN_NEG;
    return -1;
}

struct chain_builder
{
    instruction_ref sink;
    int max_depth = 0;
    std::vector<instruction_ref> externals;
    std::vector<instruction_ref> absorbed;
    std::vector<int64_t> steps;
    bool save_live = false;
    bool failed    = false;

    bool fusable(instruction_ref x) const
    {
        if(binary_code(x->name()) < 0 and unary_code(x->name()) < 0)
            return false;
        if(x->get_shape().type() != shape::float_type or x->get_shape().lens() != sink->get_shape().lens())
            return false;
        return std::all_of(x->inputs().begin(), x->inputs().end(), [&](instruction_ref i) {
            return i->get_shape().type() == shape::float_type and
                   i->get_shape().lens() == sink->get_shape().lens();
        });
    }

    static bool pointwise(instruction_ref x)
    {
        return binary_code(x->name()) >= 0 or unary_code(x->name()) >= 0;
    }

    // A value with several users is computed again inside each of them when that costs one
    // operator on values that exist anyway and every user is a pointwise operator (x - mean in
    // layer normalisation, used by the variance and by the normalised value): once all of them
    // have taken it in, the tensor itself is never written.
    bool recomputed(instruction_ref x) const
    {
        if(x->outputs().size() < 2 or not fusable(x))
            return false;
        const bool cheap = std::all_of(x->inputs().begin(), x->inputs().end(), [&](instruction_ref i) {
            return not pointwise(i) or i->outputs().size() > 1;
        });
        return cheap and std::all_of(x->outputs().begin(), x->outputs().end(), [&](instruction_ref u) {
            return pointwise(u) and u->get_shape().type() == shape::float_type and
                   u->get_shape().lens() == x->get_shape().lens();
        });
    }

    bool inlined(instruction_ref x, int depth) const
    {
        if(depth > max_depth or not fusable(x))
            return false;
        return x->outputs().size() == 1 or recomputed(x);
    }

    void push(int kind, int op, int src, int reversed)
    {
        if(steps.size() / 4 >= MI355_CHAIN_MAX_STEPS)
        {
            failed = true;
            return;
        }
        steps.insert(steps.end(), {kind, op, src, reversed});
    }

    int external(instruction_ref x)
    {
        auto it = std::find(externals.begin(), externals.end(), x);
        if(it != externals.end())
            return static_cast<int>(it - externals.begin());
        int64_t sr = 0;
        int64_t sc = 0;
        if(externals.size() >= MI355_CHAIN_MAX_INPUTS or not collapse_2d(x->get_shape(), sr, sc) or
           (sc != 0 and sc != 1))
        {
            failed = true;
            return 0;
        }
        externals.push_back(x);
        return static_cast<int>(externals.size() - 1);
    }

    // leaves the value of x in the running register
    void value(instruction_ref x, int depth)
    {
        if(inlined(x, depth))
            emit(x, depth);
        else
            push(MI355_CH_LOAD, 0, external(x), 0);
    }

    void emit(instruction_ref x, int depth)
    {
        if(failed)
            return;
        if(x != sink)
            absorbed.push_back(x);
        // the operands of a recomputed value are read, not computed again in their turn
        if(x != sink and x->outputs().size() > 1)
            depth = max_depth;
        const int un = unary_code(x->name());
        if(un >= 0)
        {
            value(x->inputs()[0], depth + 1);
            push(MI355_CH_UNARY, un, 0, 0);
            return;
        }
        const int bin = binary_code(x->name());
        auto a        = x->inputs()[0];
        auto b        = x->inputs()[1];
        if(a == b)
        {
            value(a, depth + 1);
            push(MI355_CH_BINARY, bin, MI355_CH_SELF, 0);
            return;
        }
        const bool ia = inlined(a, depth + 1);
        const bool ib = inlined(b, depth + 1);
        if(ia and ib and not save_live)
        {
            emit(a, depth + 1);
            push(MI355_CH_SAVE, 0, 0, 0);
            save_live = true;
            emit(b, depth + 1);
            save_live = false;
            push(MI355_CH_BINARY, bin, MI355_CH_SAVED, 1);
        }
        else if(ia)
        {
            emit(a, depth + 1);
            push(MI355_CH_BINARY, bin, external(b), 0);
        }
        else if(ib)
        {
            emit(b, depth + 1);
            push(MI355_CH_BINARY, bin, external(a), 1);
        }
        else
        {
            push(MI355_CH_LOAD, 0, external(a), 0);
            push(MI355_CH_BINARY, bin, external(b), 0);
        }
    }
};

void fuse_chains(module& m)
{
    std::unordered_set<const instruction*> taken;
    auto order = all_instructions(m);
    for(auto it = order.rbegin(); it != order.rend(); ++it)
    {
        auto ins = *it;
        if(taken.count(&*ins) > 0)
            continue;
        if(binary_code(ins->name()) < 0 and unary_code(ins->name()) < 0)
            continue;
        // rows of fewer than four columns gain nothing from the row-wise kernel
        if(ins->get_shape().ndim() == 0 or ins->get_shape().lens().back() < 4)
            continue;
        for(int depth : {MI355_CHAIN_MAX_STEPS, 6, 3, 1})
        {
            chain_builder cb;
            cb.sink      = ins;
            cb.max_depth = depth;
            if(not cb.fusable(ins))
                break;
            cb.emit(ins, 0);
            if(cb.failed)
                continue;
            if(cb.absorbed.empty())
                break;
            for(auto a : cb.absorbed)
                taken.insert(&*a);
            auto args = cb.externals;
            args.push_back(insert_allocation(m, ins, shape{shape::float_type, ins->get_shape().lens()}));
            chain op;
            op.steps = cb.steps;
            m.replace_instruction(ins, operation{op}, args);
            break;
        }
    }
}

// ---- layer normalisation -> one kernel ---------------------------------------------------------
//
// mean = reduce_mean(x); d = x - mean; var = reduce_mean(d * d); y = d * rsqrt(var + eps) (or
// d / sqrt(var + eps)), over the last axis -- the expansion of ONNX LayerNormalization -- with an
// add / sub / mul / div that produces x for nobody else in front and the pointwise operators that
// follow y one after the other (the scale and the shift) behind: one mi355::chain_rows whose steps
// repeat these operators in their order, the two means as row-mean steps.  x is read once and only
// the last value is written; the reference fuses the same group through src/fuse_reduce.cpp:251-340.
// Runs in front of fuse_chains, which would otherwise take the pointwise parts.

std::vector<instruction_ref> distinct_users(instruction_ref i)
{
    std::vector<instruction_ref> users;
    for(auto u : i->outputs())
    {
        if(std::none_of(users.begin(), users.end(), [&](instruction_ref v) { return &*v == &*u; }))
            users.push_back(u);
    }
    return users;
}

bool only_user_is(instruction_ref i, instruction_ref u)
{
    auto users = distinct_users(i);
    return users.size() == 1 and &*users[0] == &*u;
}

bool reduce_mean_last(instruction_ref i)
{
    if(i->name() != "reduce_mean")
        return false;
    const auto& axes = any_cast<op::reduce_mean>(i->get_operator()).axes;
    const auto nd    = static_cast<int64_t>(i->inputs()[0]->get_shape().ndim());
    return axes.size() == 1 and (axes[0] == -1 or axes[0] == nd - 1);
}

bool fuse_layer_norm(module& m, instruction_ref var)
{
    if(not reduce_mean_last(var))
        return false;
    auto sq = var->inputs()[0];
    if(sq->name() != "mul" or &*sq->inputs()[0] != &*sq->inputs()[1] or not only_user_is(sq, var))
        return false;
    auto d = sq->inputs()[0];
    if(d->name() != "sub")
        return false;
    auto x  = d->inputs()[0];
    auto mb = d->inputs()[1];
    if(mb->name() != "multibroadcast" or not only_user_is(mb, d))
        return false;
    auto mean = mb->inputs()[0];
    if(not reduce_mean_last(mean) or &*mean->inputs()[0] != &*x or not only_user_is(mean, mb))
        return false;
    const shape& xs = x->get_shape();
    if(xs.type() != shape::float_type or xs.ndim() == 0 or xs.lens().back() > MI355_CHAIN_ROWS_MAX_COLS or
       xs.lens().back() < 2 or d->get_shape().lens() != xs.lens() or mb->get_shape().lens() != xs.lens())
        return false;
    // var -> + eps -> rsqrt | sqrt -> broadcast over the row -> y
    auto var_users = distinct_users(var);
    if(var_users.size() != 1 or var_users[0]->name() != "add")
        return false;
    auto ve  = var_users[0];
    auto eps = &*ve->inputs()[0] == &*var ? ve->inputs()[1] : ve->inputs()[0];
    if(&*eps == &*var or eps->get_shape().lens() != var->get_shape().lens() or
       eps->get_shape().type() != shape::float_type)
        return false;
    auto ve_users = distinct_users(ve);
    if(ve_users.size() != 1 or (ve_users[0]->name() != "rsqrt" and ve_users[0]->name() != "sqrt"))
        return false;
    auto root        = ve_users[0];
    const bool recip = root->name() == "rsqrt";
    auto root_users  = distinct_users(root);
    if(root_users.size() != 1 or root_users[0]->name() != "multibroadcast" or
       root_users[0]->get_shape().lens() != xs.lens())
        return false;
    auto rb       = root_users[0];
    auto rb_users = distinct_users(rb);
    if(rb_users.size() != 1)
        return false;
    auto y = rb_users[0];
    if(recip ? (y->name() != "mul" or not((&*y->inputs()[0] == &*d and &*y->inputs()[1] == &*rb) or
                                          (&*y->inputs()[0] == &*rb and &*y->inputs()[1] == &*d)))
             : (y->name() != "div" or &*y->inputs()[0] != &*d or &*y->inputs()[1] != &*rb))
        return false;
    // d feeds the square and y, nothing else
    auto d_users = distinct_users(d);
    if(d_users.size() != 2 or not std::all_of(d_users.begin(), d_users.end(), [&](instruction_ref u) {
           return &*u == &*sq or &*u == &*y;
       }))
        return false;

    std::vector<instruction_ref> externals;
    std::vector<int64_t> steps;
    bool failed   = false;
    auto per_row  = var->get_shape().lens();
    auto external = [&](instruction_ref e) {
        for(std::size_t i = 0; i < externals.size(); i++)
        {
            if(&*externals[i] == &*e)
                return static_cast<int>(i);
        }
        int64_t sr = 0;
        int64_t sc = 0;
        const shape& es = e->get_shape();
        if(externals.size() >= MI355_CHAIN_MAX_INPUTS or es.type() != shape::float_type or
           (es.lens() != xs.lens() and es.lens() != per_row) or not collapse_2d(es, sr, sc) or (sc != 0 and sc != 1))
        {
            failed = true;
            return 0;
        }
        externals.push_back(e);
        return static_cast<int>(externals.size() - 1);
    };
    auto push = [&](int kind, int op, int src, int reversed) {
        if(steps.size() / 4 >= MI355_CHAIN_MAX_STEPS)
            failed = true;
        else
            steps.insert(steps.end(), {kind, op, src, reversed});
    };
    // x itself, or the one operator that makes it when nobody else reads its result
    const int x_bin    = binary_code(x->name());
    auto x_users       = distinct_users(x);
    const bool x_taken = x_bin >= 0 and x_users.size() == 2 and &*x->inputs()[0] != &*x->inputs()[1] and
                         std::all_of(x_users.begin(), x_users.end(), [&](instruction_ref u) {
                             return &*u == &*mean or &*u == &*d;
                         }) and
                         x->inputs()[0]->get_shape().lens() == xs.lens() and
                         x->inputs()[1]->get_shape().lens() == xs.lens();
    if(x_taken)
    {
        push(MI355_CH_LOAD, 0, external(x->inputs()[0]), 0);
        push(MI355_CH_BINARY, x_bin, external(x->inputs()[1]), 0);
    }
    else
        push(MI355_CH_LOAD, 0, external(x), 0);
    push(MI355_CH_SAVE, 0, 0, 0);
    push(MI355_CH_ROW_MEAN, 0, 0, 0);
    push(MI355_CH_BINARY, MI355_BIN_SUB, MI355_CH_SAVED, 1); // x - mean
    push(MI355_CH_SAVE, 0, 0, 0);
    push(MI355_CH_BINARY, MI355_BIN_MUL, MI355_CH_SELF, 0);
    push(MI355_CH_ROW_MEAN, 0, 0, 0);
    push(MI355_CH_BINARY, MI355_BIN_ADD, external(eps), &*ve->inputs()[0] == &*var ? 0 : 1);
    push(MI355_CH_UNARY, recip ? MI355_UN_RSQRT : MI355_UN_SQRT, 0, 0);
    // y = d (op) root: the saved value is the first operand, unless the graph has the product the other way round
    push(MI355_CH_BINARY, recip ? MI355_BIN_MUL : MI355_BIN_DIV, MI355_CH_SAVED, &*y->inputs()[0] == &*d ? 1 : 0);
    if(failed)
        return false;
    // what follows y one operator at a time
    auto last = y;
    while(true)
    {
        auto users = distinct_users(last);
        if(users.size() != 1)
            break;
        auto u = users[0];
        if(u->get_shape().type() != shape::float_type or u->get_shape().lens() != xs.lens())
            break;
        const auto saved_steps     = steps;
        const auto saved_externals = externals;
        const int un               = unary_code(u->name());
        const int bin              = binary_code(u->name());
        if(un >= 0)
            push(MI355_CH_UNARY, un, 0, 0);
        else if(bin >= 0 and &*u->inputs()[0] == &*u->inputs()[1])
            push(MI355_CH_BINARY, bin, MI355_CH_SELF, 0);
        else if(bin >= 0)
        {
            const bool first = &*u->inputs()[0] == &*last;
            push(MI355_CH_BINARY, bin, external(first ? u->inputs()[1] : u->inputs()[0]), first ? 0 : 1);
        }
        else
            break;
        if(failed)
        {
            steps     = saved_steps;
            externals = saved_externals;
            break;
        }
        last = u;
    }
    auto args = externals;
    args.push_back(insert_allocation(m, last, shape{shape::float_type, xs.lens()}));
    chain_rows op;
    op.steps = steps;
    m.replace_instruction(last, operation{op}, args);
    return true;
}

void fuse_layer_norms(module& m)
{
    for(auto ins : all_instructions(m))
    {
        if(ins->name() == "reduce_mean" and not ins->outputs().empty())
            fuse_layer_norm(m, ins);
    }
}

// contiguous(x) read only by float dots that take x as it lies (a 4-D view: two batch axes with a
// stride each), directly or through a transpose of the last two axes (the keys of an attention
// layer): the dots read x, the copy goes (what src/eliminate_contiguous.cpp does when the
// reader's compute_shape accepts the view).  Runs before the dots are lowered.
void skip_copies_in_front_of_dots(module& m)
{
    auto only_dots = [](instruction_ref i) {
        auto users = i->outputs();
        return not users.empty() and
               std::all_of(users.begin(), users.end(), [](instruction_ref u) { return u->name() == "dot"; });
    };
    auto swaps_last_two_of_four = [](instruction_ref t) {
        if(t->name() != "transpose")
            return false;
        const auto perm = any_cast<op::transpose>(t->get_operator()).permutation;
        return perm == std::vector<int64_t>{0, 1, 3, 2};
    };
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "contiguous" or ins->outputs().empty())
            continue;
        auto x = ins->inputs()[0];
        if(x->get_shape().ndim() != 4 or x->get_shape().type() != shape::float_type or
           x->get_shape().broadcasted())
            continue;
        auto users = ins->outputs();
        if(not std::all_of(users.begin(), users.end(), [&](instruction_ref u) {
               return u->name() == "dot" or (swaps_last_two_of_four(u) and only_dots(u));
           }))
            continue;
        for(auto u : users)
            instruction::replace_argument(u, ins, x);
    }
}

// dot -> transpose(0, 2, 1, 3) -> contiguous, the merge of the heads behind an attention layer's
// context: the dot writes its [batch, heads, rows, width] result into [batch, rows, heads, width]
// memory (its output buffer is the transposed view of a dense buffer of that layout), the transpose
// of that is dense already and the copy goes.  Runs behind the lowering of the single operators.
void write_dots_head_merged(module& m)
{
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "mi355::dot" or ins->get_shape().ndim() != 4 or
           ins->get_shape().type() != shape::float_type or not ins->get_shape().standard())
            continue;
        auto users = distinct_users(ins);
        if(users.size() != 1 or users[0]->name() != "transpose" or
           any_cast<op::transpose>(users[0]->get_operator()).permutation != std::vector<int64_t>{0, 2, 1, 3})
            continue;
        auto t      = users[0];
        auto copies = distinct_users(t);
        if(copies.empty() or not std::all_of(copies.begin(), copies.end(), [](instruction_ref c) {
               return c->name() == "mi355::contiguous";
           }))
            continue;
        const auto& l = ins->get_shape().lens();
        auto merged   = insert_allocation(m, ins, shape{shape::float_type, {l[0], l[2], l[1], l[3]}});
        auto view     = m.insert_instruction(ins, make_op("transpose", {{"permutation", {0, 2, 1, 3}}}), merged);
        instruction::replace_argument(ins, ins->inputs().back(), view);
        for(auto c : copies)
            m.replace_instruction(c, t);
    }
}

// A chain whose only reader is a quantizelinear to int8 with one scale (and one zero point) for the
// whole tensor -- the activations in front of a quantized layer, e.g. the GELU of a feed-forward
// block -- becomes one mi355::chain_q8: the float tensor is neither written nor read back.  Runs
// behind the lowering of the single operators (it matches mi355:: operators).
void fuse_chain_quantize(module& m)
{
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "mi355::quantizelinear" or ins->get_shape().type() != shape::int8_type)
            continue;
        auto x = ins->inputs()[0];
        if(x->name() != "mi355::chain" or x->outputs().size() != 1)
            continue;
        const auto& args = ins->inputs(); // x, scale, [zero point], out
        bool per_tensor  = args[1]->get_shape().type() == shape::float_type;
        for(std::size_t i = 1; i + 1 < args.size() and per_tensor; i++)
        {
            int64_t sr = 0, sc = 0;
            per_tensor = collapse_2d(args[i]->get_shape(), sr, sc) and sr == 0 and sc == 0;
        }
        if(not per_tensor)
            continue;
        chain_q8 op;
        op.steps          = any_cast<chain>(x->get_operator()).steps;
        op.has_zero_point = args.size() == 4;
        std::vector<instruction_ref> fused(x->inputs().begin(), x->inputs().end() - 1);
        fused.insert(fused.end(), args.begin() + 1, args.end());
        m.replace_instruction(ins, operation{op}, fused);
    }
}

// ---- quant_dot(a, b, scale_a, scale_b): block-scaled operands ----------------------------------
//
// The four-input form simplify_qdq leaves for the MX formats (src/simplify_qdq.cpp:290-357) goes
// to the block-scaled matrix-core kernel when both operands are fp8 e4m3fn tensors (what
// unpack_fp4 yields) with whole blocks of 32 along K.  An operand that comes straight out of
// unpack_fp4 along K is handed over still packed.  The kernel wants both operands K-contiguous:
// a B that is the transpose view of [.., N, K] storage is used as it is, any other B is copied
// into that layout.  The scales go in as the views they are (the kernel walks their strides and
// finds out on the device whether they are per-block powers of two); a scale that is visibly one
// value per block spread over 32 elements is passed in its compact form instead.

// x = unpack_fp4 along the last axis of a standard tensor: the packed tensor, else x itself
instruction_ref packed_fp4_source(instruction_ref x, bool& packed)
{
    packed = false;
    if(x->name() != "unpack_fp4")
        return x;
    const auto axis = any_cast<op::unpack_fp4>(x->get_operator()).axis;
    const auto nd   = static_cast<int64_t>(x->get_shape().ndim());
    auto src        = x->inputs().front();
    if((axis != -1 and axis != nd - 1) or not src->get_shape().standard())
        return x;
    packed = true;
    return src;
}

bool swaps_last_two(instruction_ref t)
{
    if(t->name() != "transpose")
        return false;
    const auto perm = any_cast<op::transpose>(t->get_operator()).permutation;
    const auto nd   = perm.size();
    if(nd < 2 or perm[nd - 1] != static_cast<int64_t>(nd - 2) or perm[nd - 2] != static_cast<int64_t>(nd - 1))
        return false;
    for(std::size_t i = 0; i + 2 < nd; i++)
        if(perm[i] != static_cast<int64_t>(i))
            return false;
    return true;
}

// s [.., rows, K] = reshape(multibroadcast{[.., rows, K/32, 32]}(unsqueeze(base [.., rows, K/32])))
bool compact_block_scale(instruction_ref s, instruction_ref& base)
{
    if(s->name() != "reshape")
        return false;
    auto mb = s->inputs().front();
    if(mb->name() != "multibroadcast")
        return false;
    auto us = mb->inputs().front();
    if(us->name() != "unsqueeze")
        return false;
    base             = us->inputs().front();
    const auto& bl   = base->get_shape().lens();
    const auto& ml   = mb->get_shape().lens();
    const auto& sl   = s->get_shape().lens();
    if(not base->get_shape().standard() or base->get_shape().type() != shape::float_type)
        return false;
    if(ml.size() != bl.size() + 1 or sl.size() != bl.size() or ml.back() != 32)
        return false;
    for(std::size_t i = 0; i < bl.size(); i++)
        if(ml[i] != bl[i])
            return false;
    for(std::size_t i = 0; i + 1 < bl.size(); i++)
        if(sl[i] != bl[i])
            return false;
    return sl.back() == bl.back() * 32;
}

bool lower_mx_dot(module& m, instruction_ref ins)
{
    auto a  = ins->inputs()[0];
    auto b  = ins->inputs()[1];
    auto sa = ins->inputs()[2];
    auto sb = ins->inputs()[3];
    const auto& as = a->get_shape();
    const auto& bs = b->get_shape();
    const std::size_t nd = as.ndim();
    if(as.type() != shape::fp8e4m3fn_type or bs.type() != shape::fp8e4m3fn_type or
       ins->get_shape().type() != shape::float_type or sa->get_shape().type() != shape::float_type or
       sb->get_shape().type() != shape::float_type)
        return false;
    const auto k = as.lens()[nd - 1];
    if(nd < 2 or k == 0 or k % 32 != 0)
        return false;
    quant_dot_mx op;
    // A
    a = packed_fp4_source(a, op.a_fp4);
    if(not a->get_shape().standard())
        a = make_standard(m, ins, a);
    // B as [.., N, K]
    instruction_ref b_nk;
    if(swaps_last_two(b))
        b_nk = b->inputs().front();
    else
    {
        std::vector<int64_t> perm(nd);
        for(std::size_t i = 0; i < nd; i++)
            perm[i] = static_cast<int64_t>(i);
        std::swap(perm[nd - 1], perm[nd - 2]);
        b_nk = m.insert_instruction(ins, make_op("transpose", {{"permutation", perm}}), b);
    }
    b_nk = packed_fp4_source(b_nk, op.b_fp4);
    if(not b_nk->get_shape().standard())
        b_nk = make_standard(m, ins, b_nk);
    // scales: compact where the graph shows the block structure, else the view itself
    instruction_ref base;
    if(compact_block_scale(sa, base))
    {
        sa            = base;
        op.sa_compact = true;
    }
    else if(not batch_collapses(sa->get_shape()))
        sa = make_standard(m, ins, sa);
    if(swaps_last_two(sb) and compact_block_scale(sb->inputs().front(), base))
    {
        sb            = base;
        op.sb_compact = true;
    }
    else if(not batch_collapses(sb->get_shape()))
        sb = make_standard(m, ins, sb);
    auto out_lens   = ins->get_shape().lens();
    auto out        = insert_allocation(m, ins, shape{shape::float_type, out_lens});
    // the workspace size depends on the sizes only
    std::vector<shape> probe = {a->get_shape(), b_nk->get_shape(), sa->get_shape(), sb->get_shape(),
                                shape{shape::uint8_type, {16}}, out->get_shape()};
    const auto d    = op.describe(probe);
    auto ws         = insert_allocation(m, ins, shape{shape::uint8_type, {mi355_quant_dot_mx_workspace_size(&d)}});
    m.replace_instruction(ins, operation{op}, {a, b_nk, sa, sb, ws, out});
    return true;
}

// ---- one operator at a time ------------------------------------------------------------------

void lower_instruction(module& m, instruction_ref ins)
{
    const auto name = ins->name();
    auto out        = [&](const shape& s) { return insert_allocation(m, ins, s); };
    auto standard_out = [&] { return out(shape{ins->get_shape().type(), ins->get_shape().lens()}); };
    if(name == "quant_dot")
    {
        if(ins->inputs().size() == 4)
        {
            // The four-input form the block-scaled kernel did not take (operands with element-wise scales, as the MX block formats
            // arrive after their scales are broadcast): float(a) * float(scale_a), the same for b,
            // then the float GEMM -- the three steps of ref_quant_gemm::compute
            // (src/targets/ref/lowering.cpp:221-242), each on its device kernel.
            auto as_float = [&](instruction_ref x) {
                if(x->get_shape().type() == shape::float_type)
                    return x;
                convert cv;
                cv.target_type = shape::float_type;
                auto xs        = make_standard(m, ins, x);
                return m.insert_instruction(ins, operation{cv}, xs, out(shape{shape::float_type, x->get_shape().lens()}));
            };
            auto scaled = [&](instruction_ref x, instruction_ref sc) {
                binary mul;
                mul.op = MI355_BIN_MUL;
                return m.insert_instruction(ins, operation{mul}, as_float(x), as_float(sc),
                                            out(shape{shape::float_type, x->get_shape().lens()}));
            };
            auto a = scaled(ins->inputs()[0], ins->inputs()[2]);
            auto b = scaled(ins->inputs()[1], ins->inputs()[3]);
            m.replace_instruction(ins, operation{dot{}}, a, b, standard_out());
            return;
        }
        auto a = ins->inputs()[0];
        auto b = ins->inputs()[1];
        if(not view_as_matrix(a->get_shape()).ok)
            a = make_standard(m, ins, a);
        if(not view_as_matrix(b->get_shape()).ok)
            b = make_standard(m, ins, b);
        quant_dot op;
        op.out_type = ins->get_shape().type();
        std::vector<instruction_ref> args = {a, b};
        add_dot_workspace(m, ins, op, args);
        args.push_back(standard_out());
        m.replace_instruction(ins, operation{op}, args);
    }
    else if(name == "quant_convolution")
    {
        if(ins->inputs().size() != 2)
            MIGRAPHX_THROW("mi355: quant_convolution with scale inputs has no kernel");
        auto op = conv_operator(ins);
        auto x  = make_standard(m, ins, ins->inputs()[0]);
        auto w  = make_standard(m, ins, ins->inputs()[1]);
        auto ws = insert_conv_workspace(m, ins, op, x, w);
        m.replace_instruction(ins, operation{op}, {x, w, ws, standard_out()});
    }
    else if(name == "dot")
    {
        auto a = ins->inputs()[0];
        auto b = ins->inputs()[1];
        // two batch axes keep a stride each (the head split of attention: no copy of q, k and v)
        if(not batch_collapses(a->get_shape()) and a->get_shape().ndim() != 4)
            a = make_standard(m, ins, a);
        if(not batch_collapses(b->get_shape()) and b->get_shape().ndim() != 4)
            b = make_standard(m, ins, b);
        dot op;
        op.fp32acc = fp32_dot_requested() and ins->get_shape().type() == shape::float_type;
        m.replace_instruction(ins, operation{op}, a, b, standard_out());
    }
    else if(name == "quantizelinear" or name == "dequantizelinear")
    {
        std::vector<instruction_ref> args;
        args.push_back(make_standard(m, ins, ins->inputs()[0]));
        for(std::size_t i = 1; i < ins->inputs().size(); i++)
            args.push_back(make_param(m, ins, ins->inputs()[i]));
        args.push_back(standard_out());
        if(name == "quantizelinear")
        {
            quantizelinear op;
            op.out_type = ins->get_shape().type();
            m.replace_instruction(ins, operation{op}, args);
        }
        else
        {
            m.replace_instruction(ins, operation{dequantizelinear{}}, args);
        }
    }
    else if(name == "unpack_int4" or name == "pack_int4")
    {
        // any axis, any view (transposed, broadcast): the kernel walks the input's strides
        const auto nd = ins->inputs()[0]->get_shape().ndim();
        auto x        = ins->inputs()[0];
        if(nd > MI355_MAX_DIMS)
            MIGRAPHX_THROW("mi355: " + name + " of more than 8 dimensions has no kernel");
        if(name == "unpack_int4")
        {
            unpack_int4 op;
            op.axis = any_cast<op::unpack_int4>(ins->get_operator()).axis;
            m.replace_instruction(ins, operation{op}, x, standard_out());
        }
        else
        {
            pack_int4 op;
            op.axis = any_cast<op::pack_int4>(ins->get_operator()).axis;
            m.replace_instruction(ins, operation{op}, x, standard_out());
        }
    }
    else if(name == "unpack_fp4" or name == "pack_fp4")
    {
        const auto nd   = static_cast<int64_t>(ins->inputs()[0]->get_shape().ndim());
        const auto axis = name == "unpack_fp4" ? any_cast<op::unpack_fp4>(ins->get_operator()).axis
                                               : any_cast<op::pack_fp4>(ins->get_operator()).axis;
        if(axis != -1 and axis != nd - 1)
            MIGRAPHX_THROW("mi355: " + name + " along an axis other than the last has no kernel");
        auto x = make_standard(m, ins, ins->inputs()[0]);
        if(name == "unpack_fp4")
        {
            m.replace_instruction(ins, operation{unpack_fp4{}}, x, standard_out());
        }
        else
        {
            if(x->get_shape().type() != shape::float_type)
            {
                convert cv;
                cv.target_type = shape::float_type;
                x = m.insert_instruction(ins, operation{cv}, x, out(shape{shape::float_type, x->get_shape().lens()}));
            }
            m.replace_instruction(ins, operation{pack_fp4{}}, x, standard_out());
        }
    }
    else if(name == "convolution" and ins->get_shape().type() == shape::float_type)
    {
        // what no quantization pass turned into quant_convolution: the float kernel (bit-exact, slow)
        const auto& ref = any_cast<op::convolution>(ins->get_operator());
        convolution op;
        op.padding  = ref.padding;
        op.stride   = ref.stride;
        op.dilation = ref.dilation;
        op.group    = ref.group;
        auto x = make_standard(m, ins, ins->inputs()[0]);
        auto w = make_standard(m, ins, ins->inputs()[1]);
        m.replace_instruction(ins, operation{op}, x, w, standard_out());
    }
    else if(name == "convert")
    {
        convert op;
        op.target_type = any_cast<op::convert>(ins->get_operator()).target_type;
        auto x         = make_standard(m, ins, ins->inputs()[0]);
        m.replace_instruction(ins, operation{op}, x, standard_out());
    }
    else if(name == "add" or name == "sub" or name == "mul" or name == "div" or name == "max" or name == "min")
    {
        binary op;
        op.op = name == "add"   ? MI355_BIN_ADD
                : name == "sub" ? MI355_BIN_SUB
                : name == "mul" ? MI355_BIN_MUL
                : name == "div" ? MI355_BIN_DIV
                : name == "max" ? MI355_BIN_MAX
                                : MI355_BIN_MIN;
        m.replace_instruction(ins, operation{op}, ins->inputs()[0], ins->inputs()[1], standard_out());
    }
    else if(name == "clip")
    {
        // op/clip.hpp:62-66: std::min(std::max(lowest, x), highest), as two launches
        binary mx, mn;
        mx.op    = MI355_BIN_MAX;
        mn.op    = MI355_BIN_MIN;
        auto low = m.insert_instruction(ins, operation{mx}, ins->inputs()[1], ins->inputs()[0], standard_out());
        m.replace_instruction(ins, operation{mn}, low, ins->inputs()[2], standard_out());
    }
    else if(name == "reduce_max" or name == "reduce_min")
    {
        if(ins->get_shape().elements() != 1)
            MIGRAPHX_THROW("mi355: " + name + " over part of the axes has no kernel");
        reduce_all op;
        op.op  = name == "reduce_max" ? 0 : 1;
        auto x = make_standard(m, ins, ins->inputs()[0]);
        m.replace_instruction(ins, operation{op}, x, standard_out());
    }
    else if(name == "erf" or name == "sqrt" or name == "rsqrt" or name == "exp" or name == "tanh" or
            name == "neg" or name == "nearbyint")
    {
        unary op;
        op.op  = name == "nearbyint" ? MI355_UN_NEARBYINT : name == "erf" ? MI355_UN_ERF
                               : (name == "sqrt" ? MI355_UN_SQRT
                                                 : (name == "rsqrt" ? MI355_UN_RSQRT
                                                                    : (name == "exp" ? MI355_UN_EXP
                                                                                     : (name == "tanh" ? MI355_UN_TANH
                                                                                                       : MI355_UN_NEG))));
        auto x = make_standard(m, ins, ins->inputs()[0]);
        m.replace_instruction(ins, operation{op}, x, standard_out());
    }
    else if(name == "reduce_mean")
    {
        const auto& axes = any_cast<op::reduce_mean>(ins->get_operator()).axes;
        const auto nd    = static_cast<int64_t>(ins->inputs()[0]->get_shape().ndim());
        if(axes.size() != 1 or (axes[0] != -1 and axes[0] != nd - 1))
            MIGRAPHX_THROW("mi355: reduce_mean over anything but the last axis has no kernel");
        auto x = make_standard(m, ins, ins->inputs()[0]);
        m.replace_instruction(ins, operation{reduce_mean{}}, x, standard_out());
    }
    else if(name == "softmax")
    {
        const auto axis = any_cast<op::softmax>(ins->get_operator()).axis;
        const auto nd   = static_cast<int64_t>(ins->inputs()[0]->get_shape().ndim());
        if(axis != -1 and axis != nd - 1)
            MIGRAPHX_THROW("mi355: softmax over anything but the last axis has no kernel");
        auto x = make_standard(m, ins, ins->inputs()[0]);
        m.replace_instruction(ins, operation{softmax{}}, x, standard_out());
    }
    else if(name == "gather")
    {
        if(any_cast<op::gather>(ins->get_operator()).axis != 0)
            MIGRAPHX_THROW("mi355: gather along an axis other than 0 has no kernel");
        auto t = make_standard(m, ins, ins->inputs()[0]);
        auto i = make_standard(m, ins, ins->inputs()[1]);
        m.replace_instruction(ins, operation{gather{}}, t, i, standard_out());
    }
    else if(name == "contiguous")
    {
        m.replace_instruction(ins, operation{contiguous{}}, ins->inputs()[0], standard_out());
    }
    else if(name == "reshape")
    {
        // the view operator only re-labels standard memory
        auto x = make_standard(m, ins, ins->inputs()[0]);
        if(x != ins->inputs()[0])
            m.replace_instruction(ins, ins->get_operator(), x);
    }
    else if(name[0] == '@' or name == "capture" or name.rfind("mi355::", 0) == 0 or
            (ins->get_operator().is_context_free() and ins->get_operator().output_alias({}) == 0))
    {
        // builtins, calibration taps, already lowered operators and views stay
    }
    else
    {
        MIGRAPHX_THROW("mi355: no kernel for operator '" + name + "'");
    }
}

// ---- compile-time evaluation of constant subgraphs, on the device -----------------------------

void fold_constants(module& m, context& ctx)
{
    migraphx::context gctx{ctx};
    std::unordered_map<const instruction*, argument> known;
    for(auto ins : all_instructions(m))
    {
        const auto name = ins->name();
        if(name == "mi355::literal")
        {
            known[&*ins] = any_cast<device_literal>(ins->get_operator()).data;
            continue;
        }
        if(name[0] == '@' or name == "capture" or name == "mi355::allocate" or
           name == "mi355::copy_to_device" or name == "mi355::copy_from_device")
            continue;
        const bool kernel_op = name.rfind("mi355::", 0) == 0;
        const auto& inputs   = ins->inputs();
        const std::size_t n  = kernel_op ? inputs.size() - 1 : inputs.size();
        if(inputs.empty())
            continue;
        bool all_known = true;
        for(std::size_t i = 0; i < n; i++)
            all_known = all_known and known.count(&*inputs[i]) > 0;
        if(not all_known)
            continue;
        std::vector<argument> args;
        for(std::size_t i = 0; i < n; i++)
            args.push_back(known.at(&*inputs[i]));
        if(not kernel_op)
        {
            // a view of a constant
            if(ins->get_operator().is_context_free())
                known[&*ins] = ins->get_operator().compute(ins->get_shape(), args);
            continue;
        }
        if(inputs.back()->name() != "mi355::allocate")
            continue;
        args.push_back(allocate_device(inputs.back()->get_shape()));
        argument result = ins->get_operator().compute(gctx, ins->get_shape(), args);
        ctx.finish();
        device_literal lit;
        lit.data     = result;
        known[&*ins] = result;
        m.replace_instruction(ins, operation{lit}, std::vector<instruction_ref>{});
    }
}

} // namespace

void lowering::apply(module& m) const
{
    if(ctx == nullptr)
        MIGRAPHX_THROW("mi355::lowering: no context");
    // 0. explicit copies that the float dots behind them do not need
    skip_copies_in_front_of_dots(m);
    dead_code_elimination{}.apply(m);
    // 1. fused patterns; what they absorb dies
    for(auto ins : all_instructions(m))
    {
        if(ins->name() == "dot")
            lower_w4a16(m, ins);
        else if(ins->name() == "quant_dot" and ins->inputs().size() == 4)
            lower_mx_dot(m, ins);
        else if(not fuse_quant_dot_dq(m, ins) and not fuse_quant_conv_dq(m, ins))
            fuse_dot_scale(m, ins);
    }
    dead_code_elimination{}.apply(m);
    fuse_shared_w4a16(m);
    dead_code_elimination{}.apply(m);
    fuse_shared_quant_dots(m);
    dead_code_elimination{}.apply(m);
    prepack_w4a16(m);
    dead_code_elimination{}.apply(m);
    if(fuse_pointwise)
    {
        fuse_layer_norms(m);
        dead_code_elimination{}.apply(m);
        fuse_chains(m);
        dead_code_elimination{}.apply(m);
    }
    // 2. everything else, one operator at a time
    for(auto ins : all_instructions(m))
        lower_instruction(m, ins);
    dead_code_elimination{}.apply(m);
    write_dots_head_merged(m);
    dead_code_elimination{}.apply(m);
    if(fuse_pointwise)
    {
        fuse_chain_quantize(m);
        dead_code_elimination{}.apply(m);
    }
    if(prepack_quant_dot_enabled())
    {
        prepack_quant_dot(m);
        dead_code_elimination{}.apply(m);
    }
    // 3. literals live in device memory
    for(auto ins : all_instructions(m))
    {
        if(ins->name() != "@literal")
            continue;
        device_literal lit;
        lit.data = to_device(ins->get_literal().get_argument());
        m.replace_instruction(ins, operation{lit}, std::vector<instruction_ref>{});
    }
    // 4. parameters and results cross the bus inside eval when asked to
    if(offload_copy)
    {
        for(auto ins : all_instructions(m))
        {
            if(ins->name() != "@param" or ins->outputs().empty())
                continue;
            auto users = ins->outputs();
            auto pos   = std::next(ins);
            auto buf   = insert_allocation(m, pos, ins->get_shape());
            auto dev   = m.insert_instruction(pos, operation{copy_to_device{}}, ins, buf);
            for(auto u : users)
                instruction::replace_argument(u, ins, dev);
        }
        auto last = std::prev(m.end());
        if(last->name() == "@return")
        {
            auto rets = last->inputs();
            for(auto r : rets)
            {
                auto h = m.insert_instruction(last, operation{copy_from_device{}}, r);
                instruction::replace_argument(last, r, h);
            }
        }
        else
        {
            m.add_instruction(operation{copy_from_device{}}, last);
        }
    }
    // 5. constant subgraphs (weight quantization, column sums) run once, now
    fold_constants(m, *ctx);
}

// ---- buffer reuse -------------------------------------------------------------------------------

void memory_coloring::apply(module& m) const
{
    const auto order = all_instructions(m);
    std::unordered_map<const instruction*, int> index;
    for(std::size_t i = 0; i < order.size(); i++)
        index[&*order[i]] = static_cast<int>(i);
    // the allocation an instruction's result lives in: its own (mi355::allocate), or that of the
    // argument it returns (device operators return their output buffer, views their input)
    std::unordered_map<const instruction*, const instruction*> root;
    struct life
    {
        instruction_ref ins;
        int first = -1, last = -1;
        std::size_t bytes = 0, offset = 0;
    };
    std::unordered_map<const instruction*, life> lives;
    const int forever = static_cast<int>(order.size());
    auto touch        = [&](const instruction* r, int at) {
        auto& l = lives.at(r);
        l.first = l.first < 0 ? at : std::min(l.first, at);
        l.last  = std::max(l.last, at);
    };
    for(std::size_t i = 0; i < order.size(); i++)
    {
        auto ins        = order[i];
        const auto name = ins->name();
        if(name == "mi355::allocate")
        {
            root[&*ins]  = &*ins;
            lives[&*ins] = life{ins, -1, -1, (std::max<std::size_t>(ins->get_shape().bytes(), 16) + 255) / 256 * 256, 0};
            continue;
        }
        std::vector<shape> in_shapes;
        for(auto x : ins->inputs())
            in_shapes.push_back(x->get_shape());
        const auto alias = ins->inputs().empty() ? -1 : ins->get_operator().output_alias(in_shapes);
        const instruction* mine = nullptr;
        if(alias >= 0 and alias < static_cast<std::ptrdiff_t>(ins->inputs().size()))
        {
            auto it = root.find(&*ins->inputs()[alias]);
            mine    = it == root.end() ? nullptr : it->second;
        }
        root[&*ins] = mine;
        // results of the program, and arguments of anything that is neither a device operator nor a
        // view (it may hand its argument on without saying so), stay for good
        const bool known = name.rfind("mi355::", 0) == 0 or (alias >= 0 and ins->get_operator().is_context_free());
        const int until  = (name == "@return" or not known) ? forever : static_cast<int>(i);
        for(auto x : ins->inputs())
        {
            auto it = root.find(&*x);
            if(it != root.end() and it->second != nullptr)
                touch(it->second, until);
        }
        // (a use marks the allocation from its own position on, whatever `until` says)
        for(auto x : ins->inputs())
        {
            auto it = root.find(&*x);
            if(it != root.end() and it->second != nullptr)
                lives.at(it->second).first = std::min(lives.at(it->second).first, static_cast<int>(i));
        }
    }
    if(not order.empty() and order.back()->name() != "@return")
    {
        auto it = root.find(&*order.back());
        if(it != root.end() and it->second != nullptr)
            touch(it->second, forever);
    }
    std::vector<life*> todo;
    for(auto& kv : lives)
    {
        if(kv.second.first < 0) // never used: dead code elimination's business
            kv.second.first = kv.second.last = index.at(kv.first);
        todo.push_back(&kv.second);
    }
    if(todo.empty())
        return;
    // largest first, each at the lowest offset that is free for the whole of its life
    std::sort(todo.begin(), todo.end(), [&](const life* a, const life* b) {
        if(a->bytes != b->bytes)
            return a->bytes > b->bytes;
        return index.at(&*a->ins) < index.at(&*b->ins);
    });
    std::vector<life*> placed;
    std::size_t total = 0;
    for(auto* l : todo)
    {
        std::vector<std::pair<std::size_t, std::size_t>> busy;
        for(auto* o : placed)
        {
            if(o->first <= l->last and l->first <= o->last)
                busy.emplace_back(o->offset, o->offset + o->bytes);
        }
        std::sort(busy.begin(), busy.end());
        std::size_t at = 0;
        for(const auto& b : busy)
        {
            if(at + l->bytes <= b.first)
                break;
            at = std::max(at, b.second);
        }
        l->offset = at;
        total     = std::max(total, at + l->bytes);
        placed.push_back(l);
    }
    arena whole;
    whole.bytes = total;
    auto block  = m.insert_instruction(m.begin(), operation{whole});
    for(auto* l : placed)
    {
        load at;
        at.s      = l->ins->get_shape();
        at.offset = l->offset;
        m.replace_instruction(l->ins, operation{at}, std::vector<instruction_ref>{block});
    }
}

} // namespace mi355
} // namespace migraphx
