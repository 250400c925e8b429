#include <migraphx/onnx.hpp>
#include <migraphx/make_op.hpp>
#include <migraphx/ops.hpp>
#include <migraphx/passes.hpp>
#include <cmath>
#include <cstring>
#include <fstream>
#include <functional>
#include <map>
#include <numeric>
#include <sstream>
#include <unordered_map>

namespace migraphx {

namespace {

// ---- protobuf wire format ----------------------------------------------------------------------
// A message is a sequence of (field number << 3 | wire type) keys, each followed by a varint (0),
// eight bytes (1), a length and that many bytes (2) or four bytes (5).
struct wire
{
    const unsigned char* p;
    const unsigned char* end;

    bool done() const { return p >= end; }

    uint64_t varint()
    {
        uint64_t r = 0;
        for(int shift = 0; shift < 64; shift += 7)
        {
            if(p >= end)
                MIGRAPHX_THROW("parse_onnx: truncated varint");
            const unsigned char b = *p++;
            r |= static_cast<uint64_t>(b & 0x7f) << shift;
            if((b & 0x80) == 0)
                return r;
        }
        MIGRAPHX_THROW("parse_onnx: varint too long");
    }

    wire bytes()
    {
        const uint64_t n = varint();
        if(n > static_cast<uint64_t>(end - p))
            MIGRAPHX_THROW("parse_onnx: length-delimited field runs past the end");
        wire r{p, p + n};
        p += n;
        return r;
    }

    std::string str()
    {
        wire w = bytes();
        return {reinterpret_cast<const char*>(w.p), static_cast<std::size_t>(w.end - w.p)};
    }

    template <class T>
    T fixed()
    {
        if(sizeof(T) > static_cast<std::size_t>(end - p))
            MIGRAPHX_THROW("parse_onnx: truncated fixed-width field");
        T v;
        std::memcpy(&v, p, sizeof(T));
        p += sizeof(T);
        return v;
    }

    // next key; false at the end of the message
    bool next(uint32_t& field, uint32_t& type)
    {
        if(done())
            return false;
        const uint64_t key = varint();
        field              = static_cast<uint32_t>(key >> 3);
        type               = static_cast<uint32_t>(key & 7);
        return true;
    }

    void skip(uint32_t type)
    {
        switch(type)
        {
        case 0: varint(); break;
        case 1: fixed<uint64_t>(); break;
        case 2: bytes(); break;
        case 5: fixed<uint32_t>(); break;
        default: MIGRAPHX_THROW("parse_onnx: unsupported wire type " + std::to_string(type));
        }
    }

    // repeated scalar field: packed (one length-delimited run) or one element per key
    template <class F>
    void repeated(uint32_t type, uint32_t element_type, F f)
    {
        if(type == 2 and element_type != 2)
        {
            wire run = bytes();
            while(not run.done())
                f(run);
        }
        else
        {
            f(*this);
        }
    }
};

// ---- the ONNX messages, reduced to the fields read here (onnx.proto field numbers) -------------
struct tensor_proto
{
    std::vector<int64_t> dims;
    int data_type = 0;
    std::string name;
    std::string raw;
    std::vector<float> floats;
    std::vector<int64_t> ints; // int32_data and int64_data
    std::vector<double> doubles;
};

struct attribute_proto
{
    std::string name;
    float f   = 0;
    int64_t i = 0;
    std::string s;
    tensor_proto t;
    std::vector<float> floats;
    std::vector<int64_t> ints;
};

struct node_proto
{
    std::vector<std::string> inputs;
    std::vector<std::string> outputs;
    std::string name;
    std::string op_type;
    std::string domain;
    std::map<std::string, attribute_proto> attributes;
};

struct value_info
{
    std::string name;
    int elem_type = 0;
    std::vector<int64_t> dims;
    bool has_shape = false;
};

tensor_proto read_tensor(wire w)
{
    tensor_proto t;
    uint32_t field = 0;
    uint32_t type  = 0;
    while(w.next(field, type))
    {
        switch(field)
        {
        case 1: w.repeated(type, 0, [&](wire& r) { t.dims.push_back(static_cast<int64_t>(r.varint())); }); break;
        case 2: t.data_type = static_cast<int>(w.varint()); break;
        case 4: w.repeated(type, 5, [&](wire& r) { t.floats.push_back(r.fixed<float>()); }); break;
        case 5:
            // int32 values are sign-extended to 64 bits on the wire
            w.repeated(type, 0, [&](wire& r) { t.ints.push_back(static_cast<int32_t>(r.varint())); });
            break;
        case 7: w.repeated(type, 0, [&](wire& r) { t.ints.push_back(static_cast<int64_t>(r.varint())); }); break;
        case 8: t.name = w.str(); break;
        case 9: t.raw = w.str(); break;
        case 10: w.repeated(type, 1, [&](wire& r) { t.doubles.push_back(r.fixed<double>()); }); break;
        case 13: MIGRAPHX_THROW("parse_onnx: tensors with external data are not supported");
        default: w.skip(type);
        }
    }
    return t;
}

attribute_proto read_attribute(wire w)
{
    attribute_proto a;
    uint32_t field = 0;
    uint32_t type  = 0;
    while(w.next(field, type))
    {
        switch(field)
        {
        case 1: a.name = w.str(); break;
        case 2: a.f = w.fixed<float>(); break;
        case 3: a.i = static_cast<int64_t>(w.varint()); break;
        case 4: a.s = w.str(); break;
        case 5: a.t = read_tensor(w.bytes()); break;
        case 7: w.repeated(type, 5, [&](wire& r) { a.floats.push_back(r.fixed<float>()); }); break;
        case 8: w.repeated(type, 0, [&](wire& r) { a.ints.push_back(static_cast<int64_t>(r.varint())); }); break;
        default: w.skip(type);
        }
    }
    return a;
}

node_proto read_node(wire w)
{
    node_proto n;
    uint32_t field = 0;
    uint32_t type  = 0;
    while(w.next(field, type))
    {
        switch(field)
        {
        case 1: n.inputs.push_back(w.str()); break;
        case 2: n.outputs.push_back(w.str()); break;
        case 3: n.name = w.str(); break;
        case 4: n.op_type = w.str(); break;
        case 5: {
            auto a               = read_attribute(w.bytes());
            n.attributes[a.name] = a;
            break;
        }
        case 7: n.domain = w.str(); break;
        default: w.skip(type);
        }
    }
    return n;
}

value_info read_value_info(wire w)
{
    value_info v;
    uint32_t field = 0;
    uint32_t type  = 0;
    while(w.next(field, type))
    {
        if(field == 1)
            v.name = w.str();
        else if(field == 2)
        {
            // TypeProto { tensor_type = 1 { elem_type = 1; shape = 2 { dim = 1 { dim_value = 1 } } } }
            wire tp = w.bytes();
            uint32_t f2 = 0, t2 = 0;
            while(tp.next(f2, t2))
            {
                if(f2 != 1)
                {
                    tp.skip(t2);
                    continue;
                }
                wire tt = tp.bytes();
                uint32_t f3 = 0, t3 = 0;
                while(tt.next(f3, t3))
                {
                    if(f3 == 1)
                        v.elem_type = static_cast<int>(tt.varint());
                    else if(f3 == 2)
                    {
                        v.has_shape = true;
                        wire sh = tt.bytes();
                        uint32_t f4 = 0, t4 = 0;
                        while(sh.next(f4, t4))
                        {
                            if(f4 != 1)
                            {
                                sh.skip(t4);
                                continue;
                            }
                            wire dim    = sh.bytes();
                            int64_t val = -1; // a symbolic or missing dimension
                            uint32_t f5 = 0, t5 = 0;
                            while(dim.next(f5, t5))
                            {
                                if(f5 == 1)
                                    val = static_cast<int64_t>(dim.varint());
                                else
                                    dim.skip(t5);
                            }
                            v.dims.push_back(val);
                        }
                    }
                    else
                        tt.skip(t3);
                }
            }
        }
        else
            w.skip(type);
    }
    return v;
}

// onnx.proto TensorProto.DataType -> shape::type_t (src/onnx/onnx_parser.cpp get_type)
shape::type_t get_type(int dtype)
{
    switch(dtype)
    {
    case 1: return shape::float_type;
    case 2: return shape::uint8_type;
    case 3: return shape::int8_type;
    case 4: return shape::uint16_type;
    case 5: return shape::int16_type;
    case 6: return shape::int32_type;
    case 7: return shape::int64_type;
    case 9: return shape::bool_type;
    case 10: return shape::half_type;
    case 11: return shape::double_type;
    case 12: return shape::uint32_type;
    case 13: return shape::uint64_type;
    case 16: return shape::bf16_type;
    case 17: return shape::fp8e4m3fn_type;
    default: MIGRAPHX_THROW("parse_onnx: unsupported tensor data type " + std::to_string(dtype));
    }
}

literal make_literal(const tensor_proto& t)
{
    const auto type = get_type(t.data_type);
    std::vector<std::size_t> lens(t.dims.begin(), t.dims.end());
    const shape s = lens.empty() ? shape{type} : shape{type, lens};
    if(not t.raw.empty())
    {
        if(t.raw.size() != s.bytes())
            MIGRAPHX_THROW("parse_onnx: raw_data of '" + t.name + "' has " + std::to_string(t.raw.size()) +
                           " bytes, the shape needs " + std::to_string(s.bytes()));
        return literal{s, t.raw.data()};
    }
    if(s.elements() == 0)
        return literal{s, std::vector<float>{}};
    switch(type)
    {
    case shape::float_type: return literal{s, t.floats};
    case shape::double_type: return literal{s, t.doubles};
    case shape::half_type:
    case shape::bf16_type:
    case shape::fp8e4m3fn_type: {
        // the typed fields hold the bit patterns of these types
        argument a{s};
        for(std::size_t i = 0; i < t.ints.size() and i < s.elements(); i++)
        {
            const auto bits = static_cast<uint16_t>(t.ints[i]);
            std::memcpy(a.data() + i * s.type_size(), &bits, s.type_size());
        }
        return literal{s, a.data()};
    }
    default: return literal{s, t.ints};
    }
}

// ---- node parsers -------------------------------------------------------------------------------
struct node_info
{
    const node_proto* node;
    module* mod;
    bool has(const std::string& a) const { return node->attributes.count(a) > 0; }
    const attribute_proto& attr(const std::string& a) const { return node->attributes.at(a); }
};

using node_parser = std::function<instruction_ref(const node_info&, const std::vector<instruction_ref>&)>;

std::string lens_string(const std::vector<std::size_t>& l)
{
    std::stringstream ss;
    for(std::size_t i = 0; i < l.size(); i++)
        ss << (i == 0 ? "" : ", ") << l[i];
    return ss.str();
}

int64_t tune_axis(std::size_t rank, int64_t axis, const std::string& op_name)
{
    if(axis < -static_cast<int64_t>(rank) or axis >= static_cast<int64_t>(rank))
        MIGRAPHX_THROW(op_name + ": axis is out of range.");
    return axis < 0 ? axis + static_cast<int64_t>(rank) : axis;
}

// scale and zero point brought to x's dimensions:
// src/op/builder/include/migraphx/op/builder/quantize_dequantize_linear.hpp:38-150
std::vector<instruction_ref> transform_qdq_inputs(
    module& m, const std::string& op_name, int64_t block_size, int64_t axis, std::vector<instruction_ref> args)
{
    const auto x_lens       = args.at(0)->get_shape().lens();
    const auto x_rank       = x_lens.size();
    const auto y_scale_lens = args.at(1)->get_shape().lens();
    auto for_params = [&](auto f) {
        for(std::size_t i = 1; i < args.size(); i++)
            args[i] = f(args[i]);
    };
    if(args.at(1)->get_shape().elements() == 1)
    {
        // one value for the tensor
        for_params([&](instruction_ref ins) {
            return m.add_instruction(make_op("multibroadcast", {{"out_lens", x_lens}}), ins);
        });
    }
    else if(y_scale_lens.size() == 1)
    {
        // one value per index of `axis`
        axis = tune_axis(x_rank, axis, op_name);
        if(x_lens[axis] != y_scale_lens[0])
            MIGRAPHX_THROW(op_name + ": For per axis granularity the length of y_scale (actual: " +
                           std::to_string(y_scale_lens[0]) + ") must be equal to size of x on axis " +
                           std::to_string(axis) + "(actual: " + std::to_string(x_lens[axis]) + ")");
        std::vector<int64_t> unsqueeze_axes(x_rank);
        std::iota(unsqueeze_axes.begin(), unsqueeze_axes.end(), 0);
        unsqueeze_axes.erase(unsqueeze_axes.begin() + axis);
        for_params([&](instruction_ref ins) {
            auto u = m.add_instruction(make_op("unsqueeze", {{"axes", unsqueeze_axes}}), ins);
            return m.add_instruction(make_op("multibroadcast", {{"out_lens", x_lens}}), u);
        });
    }
    else
    {
        // one value per block of `block_size` elements along `axis`
        axis = tune_axis(x_rank, axis, op_name);
        if(x_rank != y_scale_lens.size())
            MIGRAPHX_THROW(op_name + ": x(rank: " + std::to_string(x_rank) + ") and y_scale(rank: " +
                           std::to_string(y_scale_lens.size()) + ") must be of same rank for block granularity");
        for(std::size_t i = 0; i < x_rank; i++)
        {
            if(x_lens[i] != y_scale_lens[i] and static_cast<int64_t>(i) != axis)
                MIGRAPHX_THROW(op_name + ": x(shape: " + lens_string(x_lens) + ") and y_scale(shape: " +
                               lens_string(y_scale_lens) + ") shapes may only differ along provided axis(" +
                               std::to_string(axis) + ")");
        }
        const float di = static_cast<float>(x_lens[axis]);
        const float si = static_cast<float>(y_scale_lens[axis]);
        if(si <= 1.0f)
            MIGRAPHX_THROW(op_name + ": y_scale(shape: " + lens_string(y_scale_lens) +
                           ") must have size > 1 along provided axis(" + std::to_string(axis) +
                           ") for block granularity");
        const auto block_size_min = static_cast<int64_t>(std::ceil(di / si));
        const auto block_size_max = static_cast<int64_t>(std::ceil(di / (si - 1))) - 1;
        if(block_size == 0)
            block_size = block_size_min;
        if(block_size < block_size_min or block_size > block_size_max)
            MIGRAPHX_THROW(op_name + ": Block size(actual: " + std::to_string(block_size) +
                           ") must be within range [" + std::to_string(block_size_min) + ", " +
                           std::to_string(block_size_max) + "]");
        for_params([&](instruction_ref ins) {
            if(block_size == 1)
                return ins;
            ins          = m.add_instruction(make_op("unsqueeze", {{"axes", {axis + 1}}}), ins);
            auto bc_lens = ins->get_shape().lens();
            bc_lens[axis + 1] = static_cast<std::size_t>(block_size);
            ins = m.add_instruction(make_op("multibroadcast", {{"out_lens", bc_lens}}), ins);
            std::vector<int64_t> reshape_lens(x_lens.begin(), x_lens.end());
            reshape_lens[axis] = static_cast<int64_t>(ins->get_shape().lens()[axis]) * block_size;
            ins = m.add_instruction(make_op("reshape", {{"dims", reshape_lens}}), ins);
            if(static_cast<int64_t>(x_lens[axis]) < reshape_lens[axis]) // runt block
                ins = m.add_instruction(
                    make_op("slice", {{"axes", {axis}}, {"starts", {0}}, {"ends", {x_lens[axis]}}}), ins);
            return ins;
        });
    }
    return args;
}

// src/onnx/parse_dequantizelinear.cpp:41-81
instruction_ref parse_dequantizelinear(const node_info& info, const std::vector<instruction_ref>& args)
{
    if(args.size() < 2 or args.size() > 3)
        MIGRAPHX_THROW("DequantizeLinear: must have either 2 or 3 inputs, " + std::to_string(args.size()) +
                       " inputs provided");
    if(args.size() == 3)
    {
        if(args[0]->get_shape().type() != args[2]->get_shape().type())
            MIGRAPHX_THROW("DequantizeLinear: x and y_zero_point must be of same type");
        if(args[1]->get_shape().lens() != args[2]->get_shape().lens())
            MIGRAPHX_THROW("DequantizeLinear: y_scale and y_zero_point shape mismatch. Provided y_scale shape: " +
                           lens_string(args[1]->get_shape().lens()) + ", provided y_zero_point shape: " +
                           lens_string(args[2]->get_shape().lens()));
    }
    const int64_t axis  = info.has("axis") ? info.attr("axis").i : 1;
    const int64_t block = info.has("block_size") ? info.attr("block_size").i : 0;
    auto a = transform_qdq_inputs(*info.mod, "dequantizelinear", block, axis, args);
    return info.mod->add_instruction(make_op("dequantizelinear"), a);
}

// src/onnx/parse_quantizelinear.cpp:40-100, src/op/builder/quantizelinear.cpp:86-116
instruction_ref parse_quantizelinear(const node_info& info, const std::vector<instruction_ref>& args)
{
    if(args.size() < 2 or args.size() > 3)
        MIGRAPHX_THROW("QuantizeLinear: must have either 2 or 3 inputs, " + std::to_string(args.size()) +
                       " input(s) provided");
    if(args.size() == 3 and args[1]->get_shape().lens() != args[2]->get_shape().lens())
        MIGRAPHX_THROW("QuantizeLinear: y_scale and y_zero_point shapes must be equal. Provided y_scale shape: " +
                       lens_string(args[1]->get_shape().lens()) + ", provided y_zero_point shape: " +
                       lens_string(args[2]->get_shape().lens()));
    const int64_t axis  = info.has("axis") ? info.attr("axis").i : 1;
    const int64_t block = info.has("block_size") ? info.attr("block_size").i : 0;
    int64_t out_type    = -1;
    if(info.has("output_dtype"))
    {
        out_type = get_type(static_cast<int>(info.attr("output_dtype").i));
        if(args.size() == 3 and static_cast<shape::type_t>(out_type) != args[2]->get_shape().type())
            MIGRAPHX_THROW("QuantizeLinear: output_type and y_zero_point type must match.");
    }
    auto a = transform_qdq_inputs(*info.mod, "quantizelinear", block, axis, args);
    // x and the scale in one type (float wins over half)
    const auto tx = a[0]->get_shape().type();
    const auto ts = a[1]->get_shape().type();
    if(tx != ts)
    {
        const auto common = (tx == shape::float_type or ts == shape::float_type) ? shape::float_type : tx;
        for(int i = 0; i < 2; i++)
        {
            if(a[i]->get_shape().type() != common)
                a[i] = info.mod->add_instruction(make_op("convert", {{"target_type", common}}), a[i]);
        }
    }
    if(out_type >= 0)
        return info.mod->add_instruction(make_op("quantizelinear", {{"out_type", out_type}}), a);
    return info.mod->add_instruction(make_op("quantizelinear"), a);
}

// numpy matmul: a vector operand is a one-row / one-column matrix, leading dimensions broadcast
// (src/onnx/parse_matmul.cpp:205-330, src/op/builder/include/migraphx/op/builder/broadcast_dimensions.hpp)
instruction_ref parse_matmul(const node_info& info, const std::vector<instruction_ref>& args)
{
    if(args.size() != 2)
        MIGRAPHX_THROW("MatMul: two inputs expected");
    module& m   = *info.mod;
    auto a0     = args[0];
    auto a1     = args[1];
    const bool v0 = a0->get_shape().ndim() == 1;
    const bool v1 = a1->get_shape().ndim() == 1;
    if(v0)
        a0 = m.add_instruction(make_op("unsqueeze", {{"axes", {0}}}), a0);
    if(v1)
        a1 = m.add_instruction(make_op("unsqueeze", {{"axes", {1}}}), a1);
    auto l0 = a0->get_shape().lens();
    auto l1 = a1->get_shape().lens();
    if(not std::equal(l0.rbegin() + 2, l0.rend(), l1.rbegin() + 2, l1.rend()))
    {
        std::vector<std::size_t> b0(l0.begin(), l0.end() - 2);
        std::vector<std::size_t> b1(l1.begin(), l1.end() - 2);
        // broadcast the batch dimensions right-aligned
        const std::size_t nb = std::max(b0.size(), b1.size());
        std::vector<std::size_t> out(nb, 1);
        for(std::size_t i = 0; i < nb; i++)
        {
            const std::size_t d0 = i < nb - b0.size() ? 1 : b0[i - (nb - b0.size())];
            const std::size_t d1 = i < nb - b1.size() ? 1 : b1[i - (nb - b1.size())];
            if(d0 != d1 and d0 != 1 and d1 != 1)
                MIGRAPHX_THROW("MatMul: batch dimensions {" + lens_string(b0) + "} and {" + lens_string(b1) +
                               "} do not broadcast");
            out[i] = std::max(d0, d1);
        }
        auto n0 = out;
        n0.insert(n0.end(), l0.end() - 2, l0.end());
        auto n1 = out;
        n1.insert(n1.end(), l1.end() - 2, l1.end());
        if(l0 != n0)
            a0 = m.add_instruction(make_op("multibroadcast", {{"out_lens", n0}}), a0);
        if(l1 != n1)
            a1 = m.add_instruction(make_op("multibroadcast", {{"out_lens", n1}}), a1);
    }
    auto r = m.add_instruction(make_op("dot"), a0, a1);
    const auto nd = static_cast<int64_t>(r->get_shape().ndim());
    if(v0)
        r = m.add_instruction(make_op("squeeze", {{"axes", {nd - 2}}}), r);
    if(v1)
        r = m.add_instruction(make_op("squeeze", {{"axes", {v0 ? nd - 2 : nd - 1}}}), r);
    return r;
}

// src/onnx/parse_matmulnbits.cpp:42-126
instruction_ref parse_matmulnbits(const node_info& info, const std::vector<instruction_ref>& args)
{
    if(args.size() < 3 or args.size() > 4)
        MIGRAPHX_THROW("MatMulNBits: 3 or 4 inputs expected (a, b, scales, zero_points)");
    for(const char* a : {"N", "K", "bits", "block_size"})
    {
        if(not info.has(a))
            MIGRAPHX_THROW(std::string("MatMulNBits: Attribute ") + a + " is required");
    }
    const auto n     = static_cast<std::size_t>(info.attr("N").i);
    const auto k     = static_cast<std::size_t>(info.attr("K").i);
    const auto bits  = info.attr("bits").i;
    const auto block = static_cast<std::size_t>(info.attr("block_size").i);
    if(bits != 4)
        MIGRAPHX_THROW("MatMulNBits: bits only supported for value of 4, actual value " + std::to_string(bits));
    if(args[0]->get_shape().lens().back() != k)
        MIGRAPHX_THROW("MatMulNBits: Input A last dimension does not match K");
    return op::builder::matmulnbits(*info.mod, args[0], args[1], args[2],
                                    args.size() == 4 ? args[3] : info.mod->end(), n, k, block);
}

// scale and zero point spread over x: a vector along `axis`, anything else by multibroadcast
// (src/onnx/broadcast_qdq.cpp:34-63)
instruction_ref bcast_qdq(module& m,
                          const std::string& op_name,
                          instruction_ref x,
                          instruction_ref scale,
                          instruction_ref zp,
                          std::size_t axis = 0)
{
    const auto lens = x->get_shape().lens();
    auto spread     = [&](instruction_ref q) {
        if(q->get_shape().ndim() == 1 and q->get_shape().elements() > 1)
            return m.add_instruction(make_op("broadcast", {{"axis", axis}, {"out_lens", lens}}), q);
        return m.add_instruction(make_op("multibroadcast", {{"out_lens", lens}}), q);
    };
    return m.add_instruction(make_op(op_name), x, spread(scale), spread(zp));
}

// src/onnx/parse_qlinearmatmul.cpp:93-196: dequantize both operands, dot, quantize the result
instruction_ref parse_qlinearmatmul(const node_info& info, const std::vector<instruction_ref>& args)
{
    if(args.size() < 8)
        MIGRAPHX_THROW("QLINEARMATMUL: missing inputs");
    module& m = *info.mod;
    auto in_a = args[0];
    auto in_b = args[3];
    for(auto x : {in_a, in_b})
    {
        const auto t = x->get_shape().type();
        if(t != shape::int8_type and t != shape::uint8_type)
            MIGRAPHX_THROW("QLINEARMATMUL: unsupported input type");
    }
    auto lens_a = in_a->get_shape().lens();
    auto lens_b = in_b->get_shape().lens();
    if(lens_a.empty() or lens_b.empty())
        MIGRAPHX_THROW("QLINEARMATMUL: empty input");
    const bool a_vector = lens_a.size() == 1;
    const bool b_vector = lens_b.size() == 1;
    if(a_vector)
        lens_a.insert(lens_a.begin(), 1);
    if(b_vector)
        lens_b.push_back(1);
    if(lens_a.size() != lens_b.size() or lens_a.back() != *(lens_b.rbegin() + 1) or
       not std::equal(lens_a.rbegin() + 2, lens_a.rend(), lens_b.rbegin() + 2, lens_b.rend()))
        MIGRAPHX_THROW("QLINEARMATMUL: mismatched input dimensions");
    const auto nd_a = in_a->get_shape().ndim();
    auto dq_a = bcast_qdq(m, "dequantizelinear", in_a, args[1], args[2], nd_a >= 2 ? nd_a - 2 : 0);
    auto dq_b = bcast_qdq(m, "dequantizelinear", in_b, args[4], args[5], in_b->get_shape().ndim() - 1);
    if(a_vector)
        dq_a = m.add_instruction(make_op("unsqueeze", {{"axes", {0}}}), dq_a);
    if(b_vector)
        dq_b = m.add_instruction(make_op("unsqueeze", {{"axes", {1}}}), dq_b);
    auto y = m.add_instruction(make_op("dot"), dq_a, dq_b);
    if(a_vector)
        y = m.add_instruction(make_op("squeeze", {{"axes", {0}}}), y);
    else if(b_vector)
        y = m.add_instruction(make_op("squeeze", {{"axes", {1}}}), y);
    return bcast_qdq(m, "quantizelinear", y, args[6], args[7]);
}

// src/onnx/parse_convolution.cpp:49-106 with the attribute rules of src/op/builder/convolution.cpp:62-113
// and the SAME_UPPER / SAME_LOWER padding of src/pad_calc.cpp:31-53, :96-120 (static shapes)
migraphx::operation conv_operator(const node_info& info, instruction_ref x, instruction_ref w, const std::string& what)
{
    if(x->get_shape().ndim() < 3 or w->get_shape().ndim() != x->get_shape().ndim())
        MIGRAPHX_THROW(what + ": input and weights need the same rank of at least 3");
    const std::size_t kdims = x->get_shape().ndim() - 2;
    std::string auto_pad    = "NOTSET";
    if(info.has("auto_pad"))
    {
        auto_pad = info.attr("auto_pad").s;
        for(auto& ch : auto_pad)
            ch = static_cast<char>(std::toupper(static_cast<unsigned char>(ch)));
    }
    if(info.has("pads") and auto_pad != "NOTSET")
        MIGRAPHX_THROW("PARSE_CONV: auto_pad and padding cannot be specified simultaneously");
    auto attr_or = [&](const char* name, int64_t fill) {
        std::vector<int64_t> v = info.has(name) ? info.attr(name).ints : std::vector<int64_t>(kdims, fill);
        return v;
    };
    auto strides   = attr_or("strides", 1);
    auto dilations = attr_or("dilations", 1);
    auto paddings  = attr_or("pads", 0);
    if(strides.size() != kdims)
        MIGRAPHX_THROW("Inconsistent strides size, is: " + std::to_string(strides.size()) +
                       ", should be: " + std::to_string(kdims));
    if(dilations.size() != kdims)
        MIGRAPHX_THROW("Inconsistent dilations size, is: " + std::to_string(dilations.size()) +
                       ", should be: " + std::to_string(kdims));
    if(paddings.size() != kdims and paddings.size() != 2 * kdims)
        MIGRAPHX_THROW("Inconsistent paddings size, is: " + std::to_string(paddings.size()) +
                       ", should be: " + std::to_string(kdims) + " or: " + std::to_string(2 * kdims));
    if(auto_pad.find("SAME") != std::string::npos)
    {
        const bool upper = auto_pad.find("SAME_UPPER") != std::string::npos;
        paddings.assign(2 * kdims, 0);
        for(std::size_t i = 0; i < kdims; i++)
        {
            const auto in_dim  = static_cast<int64_t>(x->get_shape().lens()[i + 2]);
            const auto k_dim   = static_cast<int64_t>(w->get_shape().lens()[i + 2]);
            const auto out_dim = (in_dim + strides[i] - 1) / strides[i];
            const auto k_eff   = k_dim + (k_dim - 1) * (dilations[i] - 1);
            const auto pad     = std::max<int64_t>(0, (out_dim - 1) * strides[i] + k_eff - in_dim);
            paddings[upper ? i : i + kdims] = pad / 2;
            paddings[upper ? i + kdims : i] = pad - pad / 2;
        }
    }
    const int64_t group = info.has("group") ? info.attr("group").i : 1;
    return make_op("convolution",
                   {{"padding", paddings}, {"stride", strides}, {"dilation", dilations}, {"group", group}});
}

instruction_ref parse_conv(const node_info& info, const std::vector<instruction_ref>& args)
{
    if(args.size() < 2 or args.size() > 3)
        MIGRAPHX_THROW("Conv: two or three inputs expected");
    module& m = *info.mod;
    auto x    = args[0];
    auto w    = args[1];
    auto conv = m.add_instruction(conv_operator(info, x, w, "Conv"), x, w);
    if(args.size() == 3)
    {
        if(args[2]->get_shape().ndim() != 1 or args[2]->get_shape().lens()[0] != conv->get_shape().lens()[1])
            MIGRAPHX_THROW("Conv: the bias must be a vector with one value per output channel");
        auto b = m.add_instruction(make_op("broadcast", {{"axis", 1}, {"out_lens", conv->get_shape().lens()}}), args[2]);
        return m.add_instruction(make_op("add"), conv, b);
    }
    return conv;
}

// src/onnx/parse_qlinearconv.cpp:84-250: dequantize the input and the weights, convolution, the
// int32 bias dequantized with scale_x * scale_w and added, the result quantized
instruction_ref parse_qlinearconv(const node_info& info, const std::vector<instruction_ref>& args)
{
    if(args.size() < 8)
        MIGRAPHX_THROW("QLINEARCONV: missing inputs");
    module& m = *info.mod;
    auto in_x = args[0];
    auto in_w = args[3];
    for(auto x : {in_x, in_w})
    {
        const auto t = x->get_shape().type();
        if(t != shape::int8_type and t != shape::uint8_type)
            MIGRAPHX_THROW(x == in_x ? "QLINEARCONV: unsupported input type" : "QLINEARCONV: unsupported weight type");
    }
    if(args[1]->get_shape().type() != shape::float_type)
        MIGRAPHX_THROW("QLINEARCONV x scale type should be float");
    if(args[4]->get_shape().type() != shape::float_type)
        MIGRAPHX_THROW("QLINEARCONV: wt scale type should be float");
    if(args[6]->get_shape().type() != shape::float_type)
        MIGRAPHX_THROW("QLINEARCONV: y scale type should be float");
    if(args.size() > 8 and args[8]->get_shape().type() != shape::int32_type)
        MIGRAPHX_THROW("QLINEARCONV y bias should be int32");
    auto dq_x = bcast_qdq(m, "dequantizelinear", in_x, args[1], args[2]);
    auto dq_w = bcast_qdq(m, "dequantizelinear", in_w, args[4], args[5]);
    auto y    = m.add_instruction(conv_operator(info, in_x, in_w, "QLINEARCONV"), dq_x, dq_w);
    if(args.size() > 8)
    {
        auto sx = m.add_instruction(make_op("multibroadcast", {{"out_lens", args[4]->get_shape().lens()}}), args[1]);
        auto bs = m.add_instruction(make_op("mul"), sx, args[4]);
        auto db = m.add_instruction(make_op("dequantizelinear"), args[8], bs);
        auto bb = m.add_instruction(make_op("broadcast", {{"axis", 1}, {"out_lens", y->get_shape().lens()}}), db);
        auto fb = m.add_instruction(make_op("convert", {{"target_type", y->get_shape().type()}}), bb);
        y       = m.add_instruction(make_op("add"), y, fb);
    }
    return bcast_qdq(m, "quantizelinear", y, args[6], args[7]);
}

// numpy broadcasting of the two operands, then the operator (src/common.cpp insert_common_op /
// src/onnx/onnx_parser.cpp add_broadcastable_binary_op)
instruction_ref common_binary(module& m, const std::string& op, instruction_ref a, instruction_ref b,
                              const std::string& what)
{
    if(a->get_shape().lens() != b->get_shape().lens())
    {
        const auto la = a->get_shape().lens();
        const auto lb = b->get_shape().lens();
        const std::size_t nd = std::max(la.size(), lb.size());
        std::vector<std::size_t> out(nd, 1);
        for(std::size_t i = 0; i < nd; i++)
        {
            const std::size_t da = i < nd - la.size() ? 1 : la[i - (nd - la.size())];
            const std::size_t db = i < nd - lb.size() ? 1 : lb[i - (nd - lb.size())];
            if(da != db and da != 1 and db != 1)
                MIGRAPHX_THROW(what + ": shapes {" + lens_string(la) + "} and {" + lens_string(lb) +
                               "} do not broadcast");
            out[i] = std::max(da, db);
        }
        if(la != out)
            a = m.add_instruction(make_op("multibroadcast", {{"out_lens", out}}), a);
        if(lb != out)
            b = m.add_instruction(make_op("multibroadcast", {{"out_lens", out}}), b);
    }
    return m.add_instruction(make_op(op), a, b);
}

instruction_ref parse_binary(const std::string& op, const node_info& info, const std::vector<instruction_ref>& args)
{
    if(args.size() != 2)
        MIGRAPHX_THROW(info.node->op_type + ": two inputs expected");
    return common_binary(*info.mod, op, args[0], args[1], info.node->op_type);
}

// ---- MatMulInteger / MatMulIntegerToFloat (src/onnx/parse_matmul.cpp:36-330) ---------------------

// a zero point that changes nothing: all zeros, or all 128 for uint8 (which is shifted to int8)
bool is_symmetric_zero_point(instruction_ref zp)
{
    if(not zp->can_eval())
        return false;
    const double neutral = zp->get_shape().type() == shape::uint8_type ? 128.0 : 0.0;
    const auto v         = zp->eval().to_vector<double>();
    return std::all_of(v.begin(), v.end(), [&](double x) { return x == neutral; });
}

// src/op/builder/bias_uint8.cpp:49-100: uint8 data (and its zero point) move to int8 through half,
// the zero point is subtracted in the data's type; returns {data, data - zero point}
std::pair<instruction_ref, instruction_ref>
bias_uint8(module& m, instruction_ref arg, instruction_ref bias_arg, bool has_bias, const std::string& what)
{
    auto shift = [&](instruction_ref x) {
        auto offset = m.add_literal(literal{shape{shape::half_type}, std::vector<float>{-128.0f}});
        auto h      = m.add_instruction(make_op("convert", {{"target_type", shape::half_type}}), x);
        auto moved  = common_binary(m, "add", h, offset, what);
        return m.add_instruction(make_op("convert", {{"target_type", shape::int8_type}}), moved);
    };
    if(arg->get_shape().type() == shape::uint8_type)
    {
        arg      = shift(arg);
        bias_arg = has_bias ? shift(bias_arg) : arg;
    }
    if(has_bias)
        bias_arg = common_binary(m, "sub", arg, bias_arg, what);
    return {arg, bias_arg};
}

instruction_ref parse_matmul_integer(const node_info& info, const std::vector<instruction_ref>& args, bool scaled)
{
    const std::string op_name = scaled ? "quant_dot_scaled" : "quant_dot";
    module& m = *info.mod;
    if(args.size() < 2)
        MIGRAPHX_THROW(op_name + ": two operands expected");
    auto a0 = args[0];
    auto a1 = args[1];
    const bool a_prepended = a0->get_shape().ndim() == 1;
    const bool b_appended  = a1->get_shape().ndim() == 1;
    if(a_prepended)
        a0 = m.add_instruction(make_op("unsqueeze", {{"axes", {0}}}), a0);
    if(b_appended)
        a1 = m.add_instruction(make_op("unsqueeze", {{"axes", {1}}}), a1);

    std::size_t a0_zp_index = 2, a1_zp_index = 3;
    instruction_ref scale_a0, scale_a1;
    auto scale_arg = [&](instruction_ref mat, std::size_t index) {
        if(args.size() <= index)
            MIGRAPHX_THROW("PARSE_QUANT_DOT_SCALED: missing scale");
        auto sc        = args[index];
        const auto& ss = sc->get_shape();
        if(ss.type() != shape::float_type and ss.type() != shape::half_type)
            MIGRAPHX_THROW("PARSE_QUANT_DOT_SCALED: Scales must be float or half_type");
        if(ss.lens().at(0) != mat->get_shape().lens().back() and not ss.scalar())
            MIGRAPHX_THROW("PARSE_QUANT_DOT_SCALED: Scale must have same dim as matrix column");
        if(ss.lens().size() > 1 and not ss.scalar())
            MIGRAPHX_THROW("PARSE_QUANT_DOT_SCALED: Scales shape must be scalar or 1-D tensor");
        return sc;
    };
    if(scaled)
    {
        a0_zp_index = 4;
        a1_zp_index = 5;
        scale_a0    = scale_arg(a0, 2);
        scale_a1    = scale_arg(a1, 3);
        if(scale_a0->get_shape().type() != scale_a1->get_shape().type())
            MIGRAPHX_THROW(op_name + ": Scales must be the same type");
    }
    // the zero point of an operand, or the operand itself when it has none that matters
    auto bias_arg = [&](std::size_t index, instruction_ref input, bool& has) {
        has = false;
        if(args.size() <= index)
            return input;
        auto b = args[index];
        if(b->get_shape().type() != input->get_shape().type())
            MIGRAPHX_THROW(op_name + ": zero point must be the same type as data");
        if(is_symmetric_zero_point(b))
            return input;
        has = true;
        return b;
    };
    bool has_ba0 = false, has_ba1 = false, has_scale_bias = false;
    auto ba0 = bias_arg(a0_zp_index, a0, has_ba0);
    auto ba1 = bias_arg(a1_zp_index, a1, has_ba1);
    instruction_ref scaled_bias;
    if(scaled and args.size() > 6)
    {
        scaled_bias    = args[6];
        const auto& bs = scaled_bias->get_shape();
        if(bs.type() != shape::float_type and bs.type() != shape::half_type)
            MIGRAPHX_THROW("PARSE_QUANT_DOT_SCALED: Bias must be float or half_type");
        if(bs.type() != scale_a1->get_shape().type())
            MIGRAPHX_THROW("PARSE_QUANT_DOT_SCALED: Bias must be the same type as scales");
        if(bs.lens().at(0) != a1->get_shape().lens().back())
            MIGRAPHX_THROW("PARSE_QUANT_DOT_SCALED: Bias have same dim as matrix B column");
        has_scale_bias = true;
    }
    for(auto x : {a0, a1})
    {
        const auto t = x->get_shape().type();
        if(t != shape::uint8_type and t != shape::int8_type)
            MIGRAPHX_THROW(op_name + ": Unsupported type");
    }

    instruction_ref res;
    if(scaled)
    {
        // dequantize both operands (the axis is the dimension the scale's length matches, counted
        // from the back; 1 when none does), a float dot, the bias subtracted behind it
        auto dequantized = [&](instruction_ref x, instruction_ref sc, instruction_ref zp, bool no_zp) {
            const auto& lens     = x->get_shape().lens();
            const auto scale_len = sc->get_shape().lens().at(0);
            const auto rit       = std::find(lens.rbegin(), lens.rend(), scale_len);
            const int64_t axis   = rit != lens.rend() ? static_cast<int64_t>(lens.rend() - rit - 1) : 1;
            std::vector<instruction_ref> dq_args{x, sc};
            if(not no_zp)
                dq_args.push_back(zp);
            auto t = transform_qdq_inputs(m, "dequantizelinear", 0, axis, dq_args);
            return m.add_instruction(make_op("dequantizelinear"), t);
        };
        auto dq0 = dequantized(a0, scale_a0, ba0, a0 == ba0);
        auto dq1 = dequantized(a1, scale_a1, ba1, a1 == ba1);
        res      = parse_matmul(info, {dq0, dq1});
        if(has_scale_bias)
            res = common_binary(m, "sub", res, scaled_bias, op_name);
    }
    else
    {
        if(a0->get_shape().type() == shape::uint8_type or a1->get_shape().type() == shape::uint8_type)
        {
            std::tie(a0, ba0) = bias_uint8(m, a0, ba0, has_ba0, op_name);
            std::tie(a1, ba1) = bias_uint8(m, a1, ba1, has_ba1, op_name);
        }
        // src/op/builder/dot.cpp:36-44 with broadcast_dimensions.hpp:39-71: the operands with
        // their zero points taken off are multiplied -- unless the batch dimensions differ, where
        // the broadcast (of the operand as it came in) takes the place of the biased one
        const auto l0 = a0->get_shape().lens();
        const auto l1 = a1->get_shape().lens();
        if(not std::equal(l0.rbegin() + 2, l0.rend(), l1.rbegin() + 2, l1.rend()))
        {
            std::vector<std::size_t> b0(l0.begin(), l0.end() - 2), b1(l1.begin(), l1.end() - 2);
            const std::size_t nb = std::max(b0.size(), b1.size());
            std::vector<std::size_t> out(nb, 1);
            for(std::size_t i = 0; i < nb; i++)
            {
                const std::size_t d0 = i < nb - b0.size() ? 1 : b0[i - (nb - b0.size())];
                const std::size_t d1 = i < nb - b1.size() ? 1 : b1[i - (nb - b1.size())];
                if(d0 != d1 and d0 != 1 and d1 != 1)
                    MIGRAPHX_THROW(op_name + ": batch dimensions do not broadcast");
                out[i] = std::max(d0, d1);
            }
            auto n0 = out;
            n0.insert(n0.end(), l0.end() - 2, l0.end());
            auto n1 = out;
            n1.insert(n1.end(), l1.end() - 2, l1.end());
            if(l0 != n0)
                ba0 = m.add_instruction(make_op("multibroadcast", {{"out_lens", n0}}), a0);
            if(l1 != n1)
                ba1 = m.add_instruction(make_op("multibroadcast", {{"out_lens", n1}}), a1);
        }
        res = m.add_instruction(make_op("quant_dot"), ba0, ba1);
    }
    int64_t num_axis = static_cast<int64_t>(res->get_shape().ndim());
    if(a_prepended)
    {
        res = m.add_instruction(make_op("squeeze", {{"axes", {num_axis - 2}}}), res);
        --num_axis;
    }
    if(b_appended)
        res = m.add_instruction(make_op("squeeze", {{"axes", {num_axis - 1}}}), res);
    return res;
}

// ---- ConvInteger (src/onnx/parse_convolution.cpp:44-46 -> src/op/builder/convolution.cpp:185-380) ---
//
// quant_convolution(x - x_zp, w - w_zp) written out as
// conv(x, w) - conv(x_zp, w) - conv(x, w_zp) + conv(x_zp, w_zp), every term a quant_convolution of
// int8 tensors; uint8 tensors (and their zero points) move to int8 through half first, and a zero
// point that changes nothing (absent, all zeros, or all 128 for uint8) adds no term.
instruction_ref parse_convinteger(const node_info& info, const std::vector<instruction_ref>& args)
{
    if(args.size() < 2 or args.size() > 4)
        MIGRAPHX_THROW("ConvInteger: two to four inputs expected");
    module& m = *info.mod;
    auto x    = args[0];
    auto w    = args[1];
    for(auto t : {x, w})
    {
        const auto ty = t->get_shape().type();
        if(ty != shape::int8_type and ty != shape::uint8_type)
            MIGRAPHX_THROW("ConvInteger: int8 or uint8 tensors expected");
    }
    auto conv = conv_operator(info, x, w, "ConvInteger");
    auto attrs = conv.to_value();
    auto op    = make_op("quant_convolution", {{"padding", attrs.at("padding").to_vector<int64_t>()},
                                               {"stride", attrs.at("stride").to_vector<int64_t>()},
                                               {"dilation", attrs.at("dilation").to_vector<int64_t>()},
                                               {"group", attrs.at("group").to<int64_t>()}});
    auto neutral_literal = [&](instruction_ref like) {
        const float v = like->get_shape().type() == shape::uint8_type ? 128.0f : 0.0f;
        return m.add_literal(literal{shape{like->get_shape().type(), {1}, {0}}, std::vector<float>{v}});
    };
    auto zero_point = [&](instruction_ref input, std::size_t index) {
        if(args.size() <= index)
            return neutral_literal(input);
        if(input->get_shape().type() != args[index]->get_shape().type())
            MIGRAPHX_THROW("PARSE:Conv Data and Data Zero Point must have same type");
        return is_symmetric_zero_point(args[index]) ? neutral_literal(args[index]) : args[index];
    };
    auto x_zp = zero_point(x, 2);
    auto w_zp = zero_point(w, 3);
    auto shift = [&](instruction_ref v) {
        auto offset = m.add_literal(literal{shape{shape::half_type}, std::vector<float>{-128.0f}});
        auto h      = m.add_instruction(make_op("convert", {{"target_type", shape::half_type}}), v);
        auto moved  = common_binary(m, "add", h, offset, "ConvInteger");
        return m.add_instruction(make_op("convert", {{"target_type", shape::int8_type}}), moved);
    };
    if(x->get_shape().type() == shape::uint8_type)
    {
        const bool has = not is_symmetric_zero_point(x_zp);
        x              = shift(x);
        if(has)
            x_zp = shift(x_zp);
    }
    if(w->get_shape().type() == shape::uint8_type)
    {
        const bool has = not is_symmetric_zero_point(w_zp);
        w              = shift(w);
        if(has)
            w_zp = shift(w_zp);
    }
    auto ret = m.add_instruction(op, x, w);
    // the zero points spread over their tensors: x's is one value, w's one value or one per output channel
    auto spread_x = [&] { return m.add_instruction(make_op("multibroadcast", {{"out_lens", x->get_shape().lens()}}), x_zp); };
    auto spread_w = [&] {
        if(w_zp->get_shape().elements() == 1)
            return m.add_instruction(make_op("multibroadcast", {{"out_lens", w->get_shape().lens()}}), w_zp);
        return m.add_instruction(make_op("broadcast", {{"axis", 0}, {"out_lens", w->get_shape().lens()}}), w_zp);
    };
    const bool x_term = not is_symmetric_zero_point(x_zp);
    const bool w_term = not is_symmetric_zero_point(w_zp);
    if(x_term)
        ret = common_binary(m, "sub", ret, m.add_instruction(op, spread_x(), w), "ConvInteger");
    if(w_term)
        ret = common_binary(m, "sub", ret, m.add_instruction(op, x, spread_w()), "ConvInteger");
    if(x_term and w_term)
    {
        auto xs = spread_x();
        auto ws = spread_w();
        ret     = common_binary(m, "add", ret, m.add_instruction(op, xs, ws), "ConvInteger");
    }
    return ret;
}

// ---- DynamicQuantizeLinear (src/onnx/parse_dynamicquantizelinear.cpp:83-147) ----------------------
// y_scale = (max(0, max(x)) - min(0, min(x))) / 255, y_zero_point = uint8(round(clip(0 - min / y_scale,
// 0, 255))), y = quantizelinear(x, y_scale, y_zero_point): three outputs
std::vector<instruction_ref> parse_dynamicquantizelinear(const node_info& info,
                                                         const std::vector<instruction_ref>& args)
{
    if(args.size() != 1)
        MIGRAPHX_THROW("DYNAMICQUANTIZELINEAR: one input expected");
    module& m     = *info.mod;
    auto x        = args[0];
    const auto xt = x->get_shape().type();
    auto lit_0    = m.add_literal(literal{shape{xt}, std::vector<float>{0.0f}});
    std::vector<int64_t> axes(x->get_shape().ndim());
    std::iota(axes.begin(), axes.end(), 0);
    auto reduce_max_x = m.add_instruction(make_op("reduce_max", {{"axes", axes}}), x);
    auto max_x        = common_binary(m, "max", lit_0, reduce_max_x, "DynamicQuantizeLinear");
    auto reduce_min_x = m.add_instruction(make_op("reduce_min", {{"axes", axes}}), x);
    auto min_x        = common_binary(m, "min", lit_0, reduce_min_x, "DynamicQuantizeLinear");
    const auto lens   = max_x->get_shape().lens();
    const std::size_t n = max_x->get_shape().elements();
    auto q_range = m.add_literal(literal{shape{xt, lens}, std::vector<float>(n, 255.0f)});
    auto q_min   = m.add_literal(literal{shape{xt, lens}, std::vector<float>(n, 0.0f)});
    auto q_max   = m.add_literal(literal{shape{xt, lens}, std::vector<float>(n, 255.0f)});
    auto sub0    = common_binary(m, "sub", max_x, min_x, "DynamicQuantizeLinear");
    auto y_scale = common_binary(m, "div", sub0, q_range, "DynamicQuantizeLinear");
    auto div1    = common_binary(m, "div", min_x, y_scale, "DynamicQuantizeLinear");
    auto interm  = common_binary(m, "sub", q_min, div1, "DynamicQuantizeLinear");
    auto sat     = m.add_instruction(make_op("clip"), interm, q_min, q_max);
    auto round   = m.add_instruction(make_op("nearbyint"), sat);
    auto y_zp    = m.add_instruction(make_op("convert", {{"target_type", shape::uint8_type}}), round);
    auto quant   = bcast_qdq(m, "quantizelinear", x, y_scale, y_zp);
    return {quant, y_scale, y_zp};
}

using multi_parser = std::function<std::vector<instruction_ref>(const node_info&, const std::vector<instruction_ref>&)>;

// operators with several outputs
// QLinearAdd / QLinearMul (src/onnx/parse_qlinearbinary.cpp:107-161): both operands dequantized with
// their per-tensor scale and zero point, the float operation with numpy broadcasting, the result
// quantized with the output's scale and (optional) zero point.
instruction_ref parse_qlinearbinary(const std::string& op, const std::string& onnx_name, const node_info& info,
                                    const std::vector<instruction_ref>& args)
{
    if(args.size() < 7)
        MIGRAPHX_THROW(onnx_name + ": missing inputs");
    const auto ta = args[0]->get_shape().type();
    const auto tb = args[3]->get_shape().type();
    for(auto t : {ta, tb})
    {
        if(t != shape::int8_type and t != shape::uint8_type)
            MIGRAPHX_THROW(onnx_name + ": unsupported input type");
    }
    if(ta != tb)
        MIGRAPHX_THROW(onnx_name + ": mismatched input types");
    module& m = *info.mod;
    auto a    = bcast_qdq(m, "dequantizelinear", args[0], args[1], args[2]);
    auto b    = bcast_qdq(m, "dequantizelinear", args[3], args[4], args[5]);
    auto c    = common_binary(m, op, a, b, onnx_name);
    if(args.size() == 8)
        return bcast_qdq(m, "quantizelinear", c, args[6], args[7]);
    auto scale = m.add_instruction(make_op("multibroadcast", {{"out_lens", c->get_shape().lens()}}), args[6]);
    return m.add_instruction(make_op("quantizelinear"), c, scale);
}

// MatMulBnb4 (src/onnx/parse_matmulbnb4.cpp:38-275): B holds N * K 4-bit codes, two per byte, low
// nibble first, row n of the [N, K] weight after row n - 1; absmax one float per block of
// block_size consecutive codes.  quant_type 0 (FP4 there): weight = code / 8 * absmax; 1 (NF4):
// weight = table[code] * absmax.  The result is A x weight^T with the vector and batch rules of
// :249-275.  The codes index the table as int32 here (the reference converts to int64).
instruction_ref parse_matmulbnb4(const node_info& info, const std::vector<instruction_ref>& args)
{
    auto& m = *info.mod;
    auto need = [&](const char* a) {
        if(not info.has(a))
            MIGRAPHX_THROW(std::string("MatMulBnb4: Attribute ") + a + " is required but missing");
        return info.attr(a).i;
    };
    const auto n     = static_cast<std::size_t>(need("N"));
    const auto k     = static_cast<std::size_t>(need("K"));
    const auto block = need("block_size");
    if(block < 16 or (block & (block - 1)) != 0)
        MIGRAPHX_THROW("MatMulBnb4: block_size must be a power of 2 and >= 16, actual value: " +
                       std::to_string(block));
    const auto quant = need("quant_type");
    if(quant != 0 and quant != 1)
        MIGRAPHX_THROW("MatMulBnb4: quant_type must be 0 (FP4) or 1 (NF4), actual value: " + std::to_string(quant));
    if(args.size() < 3)
        MIGRAPHX_THROW("MatMulBnb4: requires exactly 3 inputs (A, B, absmax)");
    auto a             = args[0];
    const auto a_shape = a->get_shape();
    if(a_shape.scalar())
        MIGRAPHX_THROW("MatMulBnb4: Input A must have at least 1 dimension");
    if(a_shape.lens().back() != k)
        MIGRAPHX_THROW("MatMulBnb4: Input A inner dimension (" + std::to_string(a_shape.lens().back()) +
                       ") must match attribute K (" + std::to_string(k) + ")");
    const std::size_t codes = n * k, bs = static_cast<std::size_t>(block);
    const std::vector<std::size_t> b_lens{(codes + 1) / 2}, s_lens{(codes + bs - 1) / bs};
    if(args[1]->get_shape().lens() != b_lens)
        MIGRAPHX_THROW("MatMulBnb4: Input B does not match expected dims: {" + lens_string(b_lens) +
                       "}. Actual dims: {" + lens_string(args[1]->get_shape().lens()) + "}");
    if(args[2]->get_shape().lens() != s_lens)
        MIGRAPHX_THROW("MatMulBnb4: Input absmax does not match expected dims: {" + lens_string(s_lens) +
                       "}. Actual dims: {" + lens_string(args[2]->get_shape().lens()) + "}");

    auto first = [&](instruction_ref x, std::size_t have) {
        if(have > codes)
            x = m.add_instruction(make_op("slice", {{"axes", {0}}, {"starts", {0}}, {"ends", {codes}}}), x);
        return m.add_instruction(make_op("reshape", {{"dims", {n, k}}}), x);
    };
    auto w = first(m.add_instruction(make_op("unpack_int4"), args[1]), 2 * b_lens[0]);
    // every absmax repeated over its block, then cut to the N * K codes
    auto s = m.add_instruction(make_op("unsqueeze", {{"axes", {1}}}), args[2]);
    s      = m.add_instruction(make_op("multibroadcast", {{"out_lens", {s_lens[0], bs}}}), s);
    s      = first(m.add_instruction(make_op("reshape", {{"dims", {s_lens[0] * bs}}}), s), s_lens[0] * bs);
    instruction_ref value;
    if(quant == 0)
    {
        auto f     = m.add_instruction(make_op("convert", {{"target_type", shape::float_type}}), w);
        auto eight = m.add_literal(literal{shape{shape::float_type}, std::vector<float>{8.0f}});
        eight      = m.add_instruction(make_op("multibroadcast", {{"out_lens", {n, k}}}), eight);
        value      = m.add_instruction(make_op("div"), f, eight);
    }
    else
    {
        const std::vector<float> nf4 = {-1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
                                        -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
                                        0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f,
                                        0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,
                                        0.7229568362236023f, 1.0f};
        auto table = m.add_literal(literal{shape{shape::float_type, {16}}, nf4});
        auto index = m.add_instruction(make_op("convert", {{"target_type", shape::int32_type}}), w);
        value      = m.add_instruction(make_op("gather", {{"axis", 0}}), table, index);
    }
    auto wt = m.add_instruction(make_op("mul"), value, s);
    wt      = m.add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), wt);
    const auto rank = a_shape.ndim();
    if(rank == 1)
        a = m.add_instruction(make_op("unsqueeze", {{"axes", {0}}}), a);
    if(rank > 2)
    {
        auto lens = a_shape.lens();
        lens[rank - 2] = k;
        lens[rank - 1] = n;
        wt = m.add_instruction(make_op("multibroadcast", {{"out_lens", lens}}), wt);
    }
    auto out = m.add_instruction(make_op("dot"), a, wt);
    if(rank == 1)
        out = m.add_instruction(make_op("squeeze", {{"axes", {0}}}), out);
    return out;
}

// LayerNormalization (src/onnx/parse_layernorm.cpp:33-254): over the axes [axis, rank)
//   y = (x - mean) * rsqrt(variance + epsilon) * scale [+ bias], mean = reduce_mean(x),
//   variance = reduce_mean((x - mean)^2); outputs y, mean and the reciprocal standard deviation.
// 16-bit inputs are computed in float unless stash_type is 0.  The square of the differences is
// written as a product of x - mean with itself (the reference's sqdiff computes the same float).
std::vector<instruction_ref> parse_layernorm(const node_info& info, const std::vector<instruction_ref>& args)
{
    module& m          = *info.mod;
    int64_t axis       = info.has("axis") ? info.attr("axis").i : -1;
    const float eps_in = info.has("epsilon") ? info.attr("epsilon").f : 1e-5f;
    const bool stash   = info.has("stash_type") ? info.attr("stash_type").i == 1 : true;
    if(args.size() < 2 or args.size() > 3)
        MIGRAPHX_THROW("PARSE_LAYERNORM: invalid input count");
    auto valid = [](shape::type_t t, const std::string& what) {
        if(t != shape::float_type and t != shape::half_type and t != shape::bf16_type)
            MIGRAPHX_THROW("PARSE_LAYERNORM: Invalid type for " + what);
    };
    auto x          = args[0];
    const auto type = x->get_shape().type();
    const auto rank = static_cast<int64_t>(x->get_shape().ndim());
    valid(type, "input");
    if(rank < 2)
        MIGRAPHX_THROW("PARSE_LAYERNORM: invalid ndims=" + std::to_string(rank) + ", must be at least 2");
    if(axis < -rank or axis >= rank)
        MIGRAPHX_THROW("PARSE_LAYERNORM: invalid axis");
    auto scale = args[1];
    valid(scale->get_shape().type(), "scale");
    if(args.size() > 2)
        valid(args[2]->get_shape().type(), "bias");
    axis             = axis < 0 ? axis + rank : axis;
    const auto kdims = rank - axis;
    std::vector<int64_t> axes(kdims);
    std::iota(axes.begin(), axes.end(), axis);
    const bool widen = stash and type != shape::float_type;
    auto xin         = widen ? m.add_instruction(make_op("convert", {{"target_type", shape::float_type}}), x) : x;
    auto mean        = m.add_instruction(make_op("reduce_mean", {{"axes", axes}}), xin);
    auto centred     = common_binary(m, "sub", xin, mean, "LayerNormalization");
    auto variance    = m.add_instruction(make_op("reduce_mean", {{"axes", axes}}),
                                      m.add_instruction(make_op("mul"), centred, centred));
    const float eps  = type == shape::half_type and std::abs(eps_in) < 1e-7f ? 1e-7f : eps_in;
    // epsilon has the input's type (and its rounding), whatever the arithmetic is done in
    instruction_ref eps_lit = m.add_literal(literal{shape{type}, std::vector<float>{eps}});
    if(widen)
        eps_lit = m.add_instruction(make_op("convert", {{"target_type", shape::float_type}}), eps_lit);
    auto rs          = m.add_instruction(make_op("rsqrt"), common_binary(m, "add", variance, eps_lit, "LayerNormalization"));
    auto result      = common_binary(m, "mul", centred, rs, "LayerNormalization");
    if(widen)
        result = m.add_instruction(make_op("convert", {{"target_type", type}}), result);
    // a vector of scales (biases) lies along the first normalised axis
    const auto skipped = static_cast<std::size_t>(rank - kdims);
    auto along = [&](instruction_ref v) {
        if(skipped > 0 and v->get_shape().ndim() == 1)
            return m.add_instruction(make_op("broadcast", {{"axis", skipped}, {"out_lens", x->get_shape().lens()}}), v);
        return v;
    };
    auto y = common_binary(m, "mul", result, along(scale), "LayerNormalization");
    if(args.size() > 2)
        y = common_binary(m, "add", y, along(args[2]), "LayerNormalization");
    return {y, mean, rs};
}

const std::unordered_map<std::string, multi_parser>& multi_parsers()
{
    static const std::unordered_map<std::string, multi_parser> table = {
        {"DynamicQuantizeLinear", parse_dynamicquantizelinear},
        {"LayerNormalization", parse_layernorm},
    };
    return table;
}

const std::unordered_map<std::string, node_parser>& parsers()
{
    static const std::unordered_map<std::string, node_parser> table = {
        {"MatMul", parse_matmul},
        {"MatMulNBits", parse_matmulnbits},
        {"MatMulBnb4", parse_matmulbnb4},
        {"QLinearAdd", [](const node_info& i, const std::vector<instruction_ref>& a) { return parse_qlinearbinary("add", "QLinearAdd", i, a); }},
        {"QLinearMul", [](const node_info& i, const std::vector<instruction_ref>& a) { return parse_qlinearbinary("mul", "QLinearMul", i, a); }},
        {"DequantizeLinear", parse_dequantizelinear},
        {"QuantizeLinear", parse_quantizelinear},
        {"QLinearMatMul", parse_qlinearmatmul},
        {"QLinearConv", parse_qlinearconv},
        {"ConvInteger", parse_convinteger},
        {"MatMulInteger",
         [](const node_info& i, const std::vector<instruction_ref>& a) { return parse_matmul_integer(i, a, false); }},
        {"MatMulIntegerToFloat",
         [](const node_info& i, const std::vector<instruction_ref>& a) { return parse_matmul_integer(i, a, true); }},
        {"Conv", parse_conv},
        {"Add", [](const node_info& i, const std::vector<instruction_ref>& a) { return parse_binary("add", i, a); }},
        {"Sub", [](const node_info& i, const std::vector<instruction_ref>& a) { return parse_binary("sub", i, a); }},
        {"Mul", [](const node_info& i, const std::vector<instruction_ref>& a) { return parse_binary("mul", i, a); }},
        {"Div", [](const node_info& i, const std::vector<instruction_ref>& a) { return parse_binary("div", i, a); }},
        {"Identity",
         [](const node_info& i, const std::vector<instruction_ref>& a) {
             return i.mod->add_instruction(make_op("identity"), a.at(0));
         }},
        {"Transpose",
         [](const node_info& i, const std::vector<instruction_ref>& a) {
             std::vector<int64_t> perm;
             if(i.has("perm"))
                 perm = i.attr("perm").ints;
             else
             {
                 // the default reverses the dimensions
                 perm.resize(a.at(0)->get_shape().ndim());
                 std::iota(perm.rbegin(), perm.rend(), 0);
             }
             return i.mod->add_instruction(make_op("transpose", {{"permutation", perm}}), a.at(0));
         }},
        {"Reshape",
         [](const node_info& i, const std::vector<instruction_ref>& a) {
             if(a.size() != 2 or not a[1]->can_eval())
                 MIGRAPHX_THROW("Reshape: the target shape must be a constant input");
             auto dims = a[1]->eval().to_vector<int64_t>();
             // 0 keeps the input's dimension (allowzero = 0)
             for(std::size_t d = 0; d < dims.size(); d++)
             {
                 if(dims[d] == 0 and d < a[0]->get_shape().ndim())
                     dims[d] = static_cast<int64_t>(a[0]->get_shape().lens()[d]);
             }
             auto x = a[0];
             if(not x->get_shape().standard())
                 x = i.mod->add_instruction(make_op("contiguous"), x);
             return i.mod->add_instruction(make_op("reshape", {{"dims", dims}}), x);
         }},
    };
    return table;
}

program parse_model(wire model, const onnx_options& options)
{
    // ModelProto.graph = 7
    wire graph{nullptr, nullptr};
    bool found     = false;
    uint32_t field = 0;
    uint32_t type  = 0;
    while(model.next(field, type))
    {
        if(field == 7 and type == 2)
        {
            graph = model.bytes();
            found = true;
        }
        else
            model.skip(type);
    }
    if(not found)
        MIGRAPHX_THROW("parse_onnx: Failed reading onnx file.");

    std::vector<node_proto> nodes;
    std::vector<tensor_proto> initializers;
    std::vector<value_info> inputs;
    std::vector<value_info> outputs;
    while(graph.next(field, type))
    {
        switch(field)
        {
        case 1: nodes.push_back(read_node(graph.bytes())); break;
        case 5: initializers.push_back(read_tensor(graph.bytes())); break;
        case 11: inputs.push_back(read_value_info(graph.bytes())); break;
        case 12: outputs.push_back(read_value_info(graph.bytes())); break;
        default: graph.skip(type);
        }
    }

    program p;
    module* mm = p.get_main_module();
    std::unordered_map<std::string, instruction_ref> values;
    for(const auto& t : initializers)
        values[t.name] = mm->add_literal(make_literal(t));
    for(const auto& in : inputs)
    {
        if(values.count(in.name) > 0)
            continue; // an initializer listed among the inputs
        if(not in.has_shape and options.map_input_dims.count(in.name) == 0)
            MIGRAPHX_THROW("parse_onnx: input '" + in.name + "' has no shape");
        std::vector<std::size_t> lens;
        auto given = options.map_input_dims.find(in.name);
        if(given != options.map_input_dims.end())
        {
            lens = given->second;
        }
        else
        {
            // an open dimension takes the default size (onnx.cpp:50-66 of the reference: 1 unless set)
            for(auto d : in.dims)
                lens.push_back(d > 0 ? static_cast<std::size_t>(d)
                                     : std::max<std::size_t>(options.default_dim_value, 1));
        }
        const auto t    = get_type(in.elem_type);
        values[in.name] = mm->add_parameter(in.name, lens.empty() ? shape{t} : shape{t, lens});
    }
    for(const auto& n : nodes)
    {
        if(n.op_type == "Constant")
        {
            if(n.attributes.count("value") == 0)
                MIGRAPHX_THROW("Constant: only the tensor form (attribute `value`) is supported");
            values[n.outputs.at(0)] = mm->add_literal(make_literal(n.attributes.at("value").t));
            continue;
        }
        auto it    = parsers().find(n.op_type);
        auto multi = multi_parsers().find(n.op_type);
        if(it == parsers().end() and multi == multi_parsers().end())
            MIGRAPHX_THROW("parse_onnx: operator '" + n.op_type + "' is outside the quantized-GEMM path of this build");
        std::vector<instruction_ref> args;
        for(const auto& name : n.inputs)
        {
            if(name.empty())
                continue; // an omitted optional input
            if(values.count(name) == 0)
                MIGRAPHX_THROW("PARSE_GRAPH: invalid onnx file. Input \"" + name + "\" is unavailable due to unordered nodes!");
            args.push_back(values.at(name));
        }
        if(multi != multi_parsers().end())
        {
            const auto outs = multi->second(node_info{&n, mm}, args);
            for(std::size_t i = 0; i < outs.size() and i < n.outputs.size(); i++)
            {
                if(not n.outputs[i].empty())
                    values[n.outputs[i]] = outs[i];
            }
            continue;
        }
        values[n.outputs.at(0)] = it->second(node_info{&n, mm}, args);
    }
    std::vector<instruction_ref> rets;
    for(const auto& o : outputs)
    {
        if(values.count(o.name) == 0)
            MIGRAPHX_THROW("parse_onnx: graph output '" + o.name + "' is not produced by any node");
        rets.push_back(values.at(o.name));
    }
    mm->add_return(rets);
    return p;
}

} // namespace

program parse_onnx_buffer(const void* data, std::size_t size, const onnx_options& options)
{
    const auto* b = static_cast<const unsigned char*>(data);
    return parse_model(wire{b, b + size}, options);
}

program parse_onnx_buffer(const std::string& buffer, const onnx_options& options)
{
    return parse_onnx_buffer(buffer.data(), buffer.size(), options);
}

program parse_onnx(const std::string& filename, const onnx_options& options)
{
    std::ifstream is(filename, std::ios::binary);
    if(not is)
        MIGRAPHX_THROW("parse_onnx: cannot open '" + filename + "'");
    std::stringstream ss;
    ss << is.rdbuf();
    return parse_onnx_buffer(ss.str(), options);
}

} // namespace migraphx
