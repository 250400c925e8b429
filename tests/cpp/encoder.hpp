// A BERT-shaped encoder built in memory (benchmark config 5): token + position embedding,
// LayerNorm, then per layer multi-head self-attention and a GELU feed-forward block with residual
// connections and LayerNorm.  Weights ~N(0, 0.02).  In the quantized form the six projections of a
// layer (Q, K, V, O and the two feed-forward matrices) are QDQ MatMuls: int8 weights with one scale
// per output channel, activations quantized per tensor with scales from max-abs calibration; the
// attention products stay float, as does everything between the MatMuls.
#ifndef TESTS_CPP_ENCODER_HPP
#define TESTS_CPP_ENCODER_HPP

#include "common.hpp"
#include <functional>

namespace encoder {

using namespace testutil;
using migraphx::shape;

struct config
{
    std::size_t layers = 2, hidden = 128, heads = 4, ffn = 512, batch = 2, seq = 16, vocab = 100;
    std::size_t tokens() const { return batch * seq; }
};

struct linear_weights
{
    std::size_t in = 0, out = 0;
    std::vector<float> w;       // [in, out]
    std::vector<float> bias;    // [out]
    std::vector<int> wq;        // int8 values, [in, out]
    std::vector<float> wscale;  // [out]
};

struct layer_weights
{
    linear_weights q, k, v, o, f1, f2;
    std::vector<float> ln1_g, ln1_b, ln2_g, ln2_b;
};

struct weights
{
    std::vector<float> tok, pos, ln0_g, ln0_b;
    std::vector<layer_weights> layers;
};

inline linear_weights make_linear(std::size_t in, std::size_t out, unsigned seed)
{
    linear_weights l;
    l.in   = in;
    l.out  = out;
    l.w    = normal_floats(in * out, 0.02f, seed);
    l.bias = normal_floats(out, 0.02f, seed + 1);
    // symmetric per-output-channel int8: scale = max|w| / 127, q = round-to-nearest(w / scale)
    l.wscale.assign(out, 0.0f);
    for(std::size_t i = 0; i < in; i++)
        for(std::size_t o = 0; o < out; o++)
            l.wscale[o] = std::max(l.wscale[o], std::fabs(l.w[i * out + o]));
    for(auto& s : l.wscale)
        s = s == 0.0f ? 1.0f : s / 127.0f;
    l.wq.resize(in * out);
    for(std::size_t i = 0; i < in; i++)
        for(std::size_t o = 0; o < out; o++)
            l.wq[i * out + o] =
                std::max(-127, std::min(127, static_cast<int>(std::nearbyint(l.w[i * out + o] / l.wscale[o]))));
    return l;
}

inline weights make_weights(const config& c, unsigned seed)
{
    weights w;
    w.tok   = normal_floats(c.vocab * c.hidden, 0.02f, seed);
    w.pos   = normal_floats(c.seq * c.hidden, 0.02f, seed + 1);
    w.ln0_g = uniform_floats(c.hidden, 0.9f, 1.1f, seed + 2);
    w.ln0_b = normal_floats(c.hidden, 0.02f, seed + 3);
    for(std::size_t l = 0; l < c.layers; l++)
    {
        const unsigned s = seed + 100 * (l + 1);
        layer_weights lw;
        lw.q     = make_linear(c.hidden, c.hidden, s + 1);
        lw.k     = make_linear(c.hidden, c.hidden, s + 3);
        lw.v     = make_linear(c.hidden, c.hidden, s + 5);
        lw.o     = make_linear(c.hidden, c.hidden, s + 7);
        lw.f1    = make_linear(c.hidden, c.ffn, s + 9);
        lw.f2    = make_linear(c.ffn, c.hidden, s + 11);
        lw.ln1_g = uniform_floats(c.hidden, 0.9f, 1.1f, s + 13);
        lw.ln1_b = normal_floats(c.hidden, 0.02f, s + 14);
        lw.ln2_g = uniform_floats(c.hidden, 0.9f, 1.1f, s + 15);
        lw.ln2_b = normal_floats(c.hidden, 0.02f, s + 16);
        w.layers.push_back(std::move(lw));
    }
    return w;
}

// Builds the graph.  Quantized points are numbered 4*layer + {0: attention input, 1: attention
// context, 2: feed-forward input, 3: GELU output}.  With `act_scales` empty every point gets a
// `capture` operator calling `tap` (calibration graph, float MatMuls); otherwise point i is
// quantized with scale act_scales[i].
struct builder
{
    const config& c;
    const weights& w;
    std::vector<float> act_scales;
    std::function<void(std::size_t, std::vector<migraphx::argument>)> tap;
    module* mm = nullptr;

    instruction_ref lit(const std::vector<float>& v, std::vector<std::size_t> lens)
    {
        return mm->add_literal(literal{shape{shape::float_type, std::move(lens)}, v});
    }
    instruction_ref scalar_like(float v, instruction_ref x)
    {
        auto l = mm->add_literal(literal{shape{shape::float_type}, std::vector<float>{v}});
        return mm->add_instruction(make_op("multibroadcast", {{"out_lens", x->get_shape().lens()}}), l);
    }
    instruction_ref row_like(instruction_ref v, instruction_ref x) // v: [C] against x: [T, C]
    {
        return mm->add_instruction(
            make_op("broadcast", {{"axis", 1}, {"out_lens", x->get_shape().lens()}}), v);
    }
    instruction_ref col_like(instruction_ref v, instruction_ref x) // v: [T, 1] against x: [T, C]
    {
        return mm->add_instruction(make_op("multibroadcast", {{"out_lens", x->get_shape().lens()}}), v);
    }

    // reduce_mean / sub / mul / add / rsqrt, the way the ONNX LayerNormalization node is expanded
    instruction_ref layer_norm(instruction_ref x, const std::vector<float>& g, const std::vector<float>& b)
    {
        auto mean = mm->add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), x);
        auto xc   = mm->add_instruction(make_op("sub"), x, col_like(mean, x));
        auto var  = mm->add_instruction(make_op("reduce_mean", {{"axes", {-1}}}),
                                       mm->add_instruction(make_op("mul"), xc, xc));
        auto rs   = mm->add_instruction(make_op("rsqrt"),
                                      mm->add_instruction(make_op("add"), var, scalar_like(1e-5f, var)));
        auto y    = mm->add_instruction(make_op("mul"), xc, col_like(rs, x));
        y         = mm->add_instruction(make_op("mul"), y, row_like(lit(g, {g.size()}), x));
        return mm->add_instruction(make_op("add"), y, row_like(lit(b, {b.size()}), x));
    }

    // the (fake-)quantized or captured form of an activation
    instruction_ref quant_point(instruction_ref x, std::size_t point)
    {
        if(act_scales.empty())
        {
            migraphx::op::capture cap;
            cap.ins_index = point;
            cap.f         = tap;
            return mm->add_instruction(migraphx::operation{cap}, x);
        }
        auto s = mm->add_literal(literal{shape{shape::float_type}, std::vector<float>{act_scales.at(point)}});
        auto z = mm->add_literal(literal{shape{shape::int8_type}, std::vector<int>{0}});
        auto q = add_quantize_op(*mm, "quantizelinear", x, s, z);
        return add_quantize_op(*mm, "dequantizelinear", q, s, z);
    }

    instruction_ref linear(instruction_ref x, const linear_weights& l)
    {
        instruction_ref wt;
        if(act_scales.empty())
        {
            wt = lit(l.w, {l.in, l.out});
        }
        else
        {
            auto wq = mm->add_literal(literal{shape{shape::int8_type, {l.in, l.out}}, l.wq});
            auto sc = lit(l.wscale, {l.out});
            auto zp = mm->add_literal(literal{shape{shape::int8_type, {l.out}}, std::vector<int>(l.out, 0)});
            std::vector<std::size_t> wl = {l.in, l.out};
            auto scb = mm->add_instruction(make_op("broadcast", {{"axis", 1}, {"out_lens", wl}}), sc);
            auto zpb = mm->add_instruction(make_op("broadcast", {{"axis", 1}, {"out_lens", wl}}), zp);
            wt       = mm->add_instruction(make_op("dequantizelinear"), wq, scb, zpb);
        }
        auto y = mm->add_instruction(make_op("dot"), x, wt);
        return mm->add_instruction(make_op("add"), y, row_like(lit(l.bias, {l.out}), y));
    }

    // [T, H] -> [B, heads, S, d] (dense)
    instruction_ref split_heads(instruction_ref x)
    {
        const auto d = static_cast<int64_t>(c.hidden / c.heads);
        auto r = mm->add_instruction(make_op("reshape", {{"dims", {static_cast<int64_t>(c.batch), static_cast<int64_t>(c.seq), static_cast<int64_t>(c.heads), d}}}), x);
        auto t = mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 1, 3}}}), r);
        return mm->add_instruction(make_op("contiguous"), t);
    }

    instruction_ref gelu(instruction_ref x)
    {
        auto e = mm->add_instruction(make_op("erf"), mm->add_instruction(make_op("mul"), x, scalar_like(0.70710678118654752f, x)));
        auto t = mm->add_instruction(make_op("add"), e, scalar_like(1.0f, x));
        auto h = mm->add_instruction(make_op("mul"), x, scalar_like(0.5f, x));
        return mm->add_instruction(make_op("mul"), h, t);
    }

    instruction_ref layer(instruction_ref x, const layer_weights& lw, std::size_t l)
    {
        const auto d = c.hidden / c.heads;
        auto xin     = quant_point(x, 4 * l + 0);
        auto q       = split_heads(linear(xin, lw.q));
        auto k       = split_heads(linear(xin, lw.k));
        auto v       = split_heads(linear(xin, lw.v));
        auto kt      = mm->add_instruction(make_op("transpose", {{"permutation", {0, 1, 3, 2}}}), k);
        auto scores  = mm->add_instruction(make_op("dot"), q, kt);
        scores       = mm->add_instruction(make_op("mul"), scores, scalar_like(1.0f / std::sqrt(static_cast<float>(d)), scores));
        auto probs   = mm->add_instruction(make_op("softmax", {{"axis", 3}}), scores);
        auto ctx     = mm->add_instruction(make_op("dot"), probs, v);
        ctx          = mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 1, 3}}}), ctx);
        ctx          = mm->add_instruction(make_op("contiguous"), ctx);
        ctx = mm->add_instruction(make_op("reshape", {{"dims", {static_cast<int64_t>(c.tokens()), static_cast<int64_t>(c.hidden)}}}), ctx);
        auto att = linear(quant_point(ctx, 4 * l + 1), lw.o);
        auto x1  = layer_norm(mm->add_instruction(make_op("add"), x, att), lw.ln1_g, lw.ln1_b);
        auto h   = gelu(linear(quant_point(x1, 4 * l + 2), lw.f1));
        auto f   = linear(quant_point(h, 4 * l + 3), lw.f2);
        return layer_norm(mm->add_instruction(make_op("add"), x1, f), lw.ln2_g, lw.ln2_b);
    }

    program build()
    {
        program p;
        mm       = p.get_main_module();
        auto ids = mm->add_parameter("ids", shape{shape::int32_type, {c.tokens()}});
        auto tok = lit(w.tok, {c.vocab, c.hidden});
        auto x   = mm->add_instruction(make_op("gather", {{"axis", 0}}), tok, ids);
        // position embedding repeated over the batch
        auto pos = lit(w.pos, {c.seq, c.hidden});
        auto x3  = mm->add_instruction(make_op("reshape", {{"dims", {static_cast<int64_t>(c.batch), static_cast<int64_t>(c.seq), static_cast<int64_t>(c.hidden)}}}), x);
        auto pb  = mm->add_instruction(make_op("multibroadcast", {{"out_lens", x3->get_shape().lens()}}), pos);
        x3       = mm->add_instruction(make_op("add"), x3, pb);
        x        = mm->add_instruction(make_op("reshape", {{"dims", {static_cast<int64_t>(c.tokens()), static_cast<int64_t>(c.hidden)}}}), x3);
        x        = layer_norm(x, w.ln0_g, w.ln0_b);
        for(std::size_t l = 0; l < c.layers; l++)
            x = layer(x, w.layers[l], l);
        mm->add_return({x});
        return p;
    }
};

// max-abs calibration on the named target: scale of point i = max|x| / 127
inline std::vector<float>
calibrate(const config& c, const weights& w, const std::string& target_name, const argument& ids)
{
    auto t = migraphx::make_target(target_name);
    std::vector<float> amax(4 * c.layers, 0.0f);
    builder b{c, w, {}, {}};
    b.tap = [&](std::size_t i, std::vector<argument> args) {
        auto v = t.copy_from(args.front()).to_vector<float>();
        for(float x : v)
            amax[i] = std::max(amax[i], std::fabs(x));
    };
    auto p = b.build();
    p.compile(t);
    p.eval({{"ids", t.copy_to(ids)}});
    p.finish();
    for(auto& a : amax)
        a = a == 0.0f ? 1.0f : a / 127.0f;
    return amax;
}

inline program quantized(const config& c, const weights& w, const std::vector<float>& scales)
{
    builder b{c, w, scales, {}};
    return b.build();
}

} // namespace encoder
#endif
