// CPU tests of the host layer: element types, shapes, values, operator shape rules, module
// editing, registries, and the passes of the quantized-GEMM path (simplify_qdq, quantize_int8 /
// fp8 calibration, quantize_int4, the MatMulNBits graph).  Pass tests follow the reference's
// test/simplify_qdq_test.cpp, test/int4_test.cpp and test/quantization.cpp: the rewritten module
// is compared with one written out by hand, and both are evaluated on the CPU oracle target.
#include "common.hpp"
#include "encoder.hpp"
#include "oracle_target.hpp"
#include "test.hpp"
#include <sstream>
#include <migraphx/json.hpp>
#include <migraphx/load_save.hpp>
#include <migraphx/msgpack.hpp>
#include <migraphx/onnx.hpp>
#include <algorithm>
#include <fstream>

extern "C" {
float orc_fp8e4m3fn_to_f32(uint8_t x);
uint8_t orc_fp8e4m3fn_from_f32(float x);
float orc_fp8e5m2_to_f32(uint8_t x);
uint8_t orc_fp8e5m2_from_f32(float x);
uint16_t orc_half_from_f32(float x);
float orc_half_to_f32(uint16_t h);
uint16_t orc_bf16_from_f32(float x);
float orc_bf16_to_f32(uint16_t h);
}

using namespace testutil;
using migraphx::shape;

// ---------------------------------------------------------------- element types

TEST_CASE(fp8_matches_oracle)
{
    for(int c = 0; c < 256; c++)
    {
        const float a = migraphx::fp8e4m3fn::from_bits(c);
        const float b = orc_fp8e4m3fn_to_f32(c);
        EXPECT((std::isnan(a) and std::isnan(b)) or a == b);
    }
    std::mt19937 g(1);
    for(int i = 0; i < 400000; i++)
    {
        uint32_t bits = g();
        float f;
        std::memcpy(&f, &bits, 4);
        const float af = std::fabs(f);
        if(af > 464.0f and af < 512.0f)
            continue; // the reference's encoder returns NaN there; unreachable behind the clamp
        EXPECT(migraphx::fp8e4m3fn(f).bits == orc_fp8e4m3fn_from_f32(f));
    }
    for(float f : {0.0f, -0.0f, 1.0f, 1.0625f, 1.1875f, 448.0f, 1000.0f, -1000.0f, 0.001953125f, 0.0009765625f})
        EXPECT(migraphx::fp8e4m3fn(f).bits == orc_fp8e4m3fn_from_f32(f));
}

TEST_CASE(fp8e5m2_matches_oracle)
{
    for(int c = 0; c < 256; c++)
    {
        const float a = migraphx::fp8e5m2::from_bits(c);
        const float b = orc_fp8e5m2_to_f32(c);
        EXPECT((std::isnan(a) and std::isnan(b)) or (a == b and std::signbit(a) == std::signbit(b)));
        if(not std::isnan(b) and not std::isinf(b))
            EXPECT(migraphx::fp8e5m2(b).bits == c);
    }
    std::mt19937 g(2);
    for(int i = 0; i < 400000; i++)
    {
        uint32_t bits = g();
        if(i % 2 == 1) // half of the samples inside the format's range, where the rounding happens
            bits = (bits & 0x807fffffu) | ((100u + (g() % 46u)) << 23);
        float f;
        std::memcpy(&f, &bits, 4);
        EXPECT(migraphx::fp8e5m2(f).bits == orc_fp8e5m2_from_f32(f));
    }
    for(float f : {0.0f, -0.0f, 1.0f, 1.125f, 1.375f, 57344.0f, 61440.0f, 1e9f, -1e9f, 7.62939453125e-06f,
                   2.288818359375e-05f, std::numeric_limits<float>::infinity()})
        EXPECT(migraphx::fp8e5m2(f).bits == orc_fp8e5m2_from_f32(f));
    EXPECT(std::numeric_limits<migraphx::fp8e5m2>::max().bits == 0x7b);
    EXPECT(float(std::numeric_limits<migraphx::fp8e5m2>::lowest()) == -57344.0f);
    EXPECT(shape::type_size(shape::fp8e5m2_type) == 1);
    EXPECT(shape::get_type<migraphx::fp8e5m2>::value == shape::fp8e5m2_type);
}

TEST_CASE(half_bf16_match_oracle)
{
    for(int c = 0; c < 65536; c++)
    {
        const float a = migraphx::half::from_bits(c);
        const float b = orc_half_to_f32(c);
        EXPECT((std::isnan(a) and std::isnan(b)) or a == b);
        const float x = migraphx::bf16::from_bits(c);
        const float y = orc_bf16_to_f32(c);
        EXPECT((std::isnan(x) and std::isnan(y)) or x == y);
    }
    std::mt19937 g(2);
    for(int i = 0; i < 400000; i++)
    {
        uint32_t bits = g();
        float f;
        std::memcpy(&f, &bits, 4);
        if(std::isnan(f) or (std::fabs(f) < 1.2e-38f and f != 0.0f))
            continue; // NaN payloads and float subnormals are off the path
        EXPECT(migraphx::half(f).bits == orc_half_from_f32(f));
        EXPECT(migraphx::bf16(f).bits == orc_bf16_from_f32(f));
    }
    // truncation, not rounding
    EXPECT(float(migraphx::half(1.0f + 1.5f / 2048)) == 1.0f);
    EXPECT(float(migraphx::bf16(1.0f + 1.5f / 256)) == 1.0f);
    EXPECT(std::isinf(float(migraphx::half(65536.0f))));
    EXPECT(float(migraphx::half(65519.0f)) == 65504.0f);
}

// ---------------------------------------------------------------- shape, value

TEST_CASE(shape_predicates)
{
    shape s{shape::float_type, {2, 3, 4}};
    EXPECT(s.standard() and s.packed() and not s.transposed() and not s.broadcasted());
    EXPECT(s.strides() == std::vector<std::size_t>{12, 4, 1});
    EXPECT(s.elements() == 24 and s.bytes() == 96 and s.element_space() == 24);
    EXPECT(s.index({1, 2, 3}) == 23 and s.index(std::size_t{17}) == 17);
    EXPECT(s.multi(17) == std::vector<std::size_t>{1, 1, 1});

    shape t{shape::int8_type, {3, 2}, {1, 3}};
    EXPECT(t.transposed() and t.packed() and not t.standard());
    EXPECT(t.index(std::size_t{1}) == 3);

    shape b{shape::half_type, {4, 5}, {0, 1}};
    EXPECT(b.broadcasted() and not b.packed() and not b.scalar());
    EXPECT(b.element_space() == 5 and b.bytes() == 10);

    shape sc{shape::uint8_type};
    EXPECT(sc.scalar() and sc.elements() == 1 and sc.lens() == std::vector<std::size_t>{1});

    EXPECT(shape::from_permutation(shape::float_type, {2, 3}, {1, 0}).strides() ==
           std::vector<std::size_t>{1, 2});
    EXPECT(t.with_lens({5, 7}).strides() == std::vector<std::size_t>{1, 5});
    EXPECT(shape::parse_type("int8_type") == shape::int8_type);
    EXPECT(shape::type_size(shape::fp8e4m3fn_type) == 1 and shape::type_size(shape::bf16_type) == 2);
    EXPECT(test::throws([] { shape(shape::float_type, {2, 3}, {1}); }));
}

TEST_CASE(value_and_make_op)
{
    auto op = make_op("slice", {{"axes", {1}}, {"starts", {0}}, {"ends", {5}}});
    auto v  = op.to_value();
    EXPECT(v.at("axes").to_vector<int64_t>() == std::vector<int64_t>{1});
    EXPECT(v.at("ends").to_vector<int64_t>() == std::vector<int64_t>{5});
    EXPECT(op == make_op("slice", {{"ends", {5}}, {"axes", {1}}, {"starts", {0}}}));
    EXPECT(op != make_op("slice", {{"ends", {6}}, {"axes", {1}}, {"starts", {0}}}));
    EXPECT(test::throws([] { make_op("slice", {{"axis", {1}}}); }));
    EXPECT(test::throws([] { make_op("no_such_operator"); }));
    std::vector<std::size_t> lens = {2, 3};
    auto mb = make_op("multibroadcast", {{"out_lens", lens}});
    EXPECT(migraphx::any_cast<migraphx::op::multibroadcast>(mb).out_lens == lens);
    auto cv = make_op("convert", {{"target_type", shape::half_type}});
    EXPECT(migraphx::any_cast<migraphx::op::convert>(cv).target_type == shape::half_type);
    std::stringstream ss;
    ss << make_op("transpose", {{"permutation", {1, 0}}});
    EXPECT(ss.str() == "transpose[permutation=[1, 0]]");
}

// ---------------------------------------------------------------- operator shape rules

TEST_CASE(quant_dot_shapes)
{
    // src/include/migraphx/op/quant_dot.hpp:51-121
    auto qd = make_op("quant_dot");
    shape a{shape::int8_type, {4, 8}};
    shape b{shape::int8_type, {8, 6}};
    EXPECT(qd.compute_shape({a, b}) == shape{shape::int32_type, {4, 6}});
    shape af{shape::fp8e4m3fn_type, {2, 4, 8}};
    shape bf{shape::fp8e4m3fn_type, {2, 8, 6}};
    EXPECT(qd.compute_shape({af, bf}) == shape{shape::float_type, {2, 4, 6}});
    shape sa{shape::float_type, {4, 8}};
    shape sb{shape::float_type, {8, 6}};
    EXPECT(qd.compute_shape({a, b, sa, sb}).type() == shape::float_type);
    // transposed views are fine
    EXPECT(qd.compute_shape({a, shape{shape::int8_type, {8, 6}, {1, 8}}}).lens() ==
           std::vector<std::size_t>{4, 6});
    EXPECT(test::throws([&] { qd.compute_shape({a}); }));
    EXPECT(test::throws([&] { qd.compute_shape({a, shape{shape::uint8_type, {8, 6}}}); }));
    EXPECT(test::throws([&] { qd.compute_shape({a, shape{shape::int8_type, {7, 6}}}); }));
    EXPECT(test::throws([&] { qd.compute_shape({shape{shape::half_type, {4, 8}}, shape{shape::half_type, {8, 6}}}); }));
    EXPECT(test::throws([&] { qd.compute_shape({shape{shape::int8_type, {8}}, shape{shape::int8_type, {8}}}); }));
    EXPECT(test::throws([&] { qd.compute_shape({af, shape{shape::fp8e4m3fn_type, {3, 8, 6}}}); }));
    EXPECT(test::throws([&] { qd.compute_shape({a, b, sa, shape{shape::half_type, {8, 6}}}); }));
}

TEST_CASE(quant_dot_four_inputs_known_answer)
{
    // test/ref/dot_op.cpp:1836-1865 (quant_dot_4args_scales): element-wise scales, float GEMM
    program p;
    auto* mm = p.get_main_module();
    shape sa{shape::float_type, {2, 3}};
    shape sb{shape::float_type, {3, 2}};
    auto a  = mm->add_literal(literal{sa, std::vector<float>{1, 2, 3, 4, 5, 6}});
    auto b  = mm->add_literal(literal{sb, std::vector<float>{1, 2, 3, 4, 5, 6}});
    auto s1 = mm->add_literal(literal{sa, std::vector<float>{0.5f, 1, 0.5f, 1, 0.5f, 1}});
    auto s2 = mm->add_literal(literal{sb, std::vector<float>{1, 0.5f, 1, 0.5f, 1, 0.5f}});
    mm->add_return({mm->add_instruction(make_op("quant_dot"), a, b, s1, s2)});
    auto r = testutil::run_on("oracle", p, {});
    EXPECT(r.size() == 1);
    EXPECT(r[0].get_shape() == shape{shape::float_type, {2, 2}});
    EXPECT(r[0].to_vector<float>() == std::vector<float>{14.0f, 9.0f, 41.5f, 27.0f});
}

TEST_CASE(qdq_and_int4_shapes)
{
    shape x{shape::float_type, {3, 4}};
    shape zi{shape::int8_type, {3, 4}};
    EXPECT(make_op("quantizelinear").compute_shape({x, x}) == shape{shape::uint8_type, {3, 4}});
    EXPECT(make_op("quantizelinear").compute_shape({x, x, zi}) == zi);
    EXPECT(make_op("quantizelinear", {{"out_type", shape::fp8e4m3fn_type}}).compute_shape({x, x}).type() ==
           shape::fp8e4m3fn_type);
    EXPECT(test::throws([&] { make_op("quantizelinear").compute_shape({x, shape{shape::half_type, {3, 4}}}); }));
    EXPECT(test::throws([&] { make_op("quantizelinear").compute_shape({x, shape{shape::float_type, {3, 5}}}); }));
    EXPECT(make_op("dequantizelinear").compute_shape({zi, shape{shape::half_type, {3, 4}}, zi}) ==
           shape{shape::half_type, {3, 4}});
    EXPECT(test::throws([&] { make_op("dequantizelinear").compute_shape({zi, x, shape{shape::uint8_type, {3, 4}}}); }));
    shape p{shape::uint8_type, {2, 5}};
    EXPECT(make_op("unpack_int4").compute_shape({p}).lens() == std::vector<std::size_t>{2, 10});
    EXPECT(make_op("unpack_int4", {{"axis", 0}}).compute_shape({p}).lens() == std::vector<std::size_t>{4, 5});
    EXPECT(make_op("pack_int4").compute_shape({shape{shape::int8_type, {2, 6}}}).lens() ==
           std::vector<std::size_t>{2, 3});
    EXPECT(test::throws([&] { make_op("pack_int4").compute_shape({p}); })); // odd axis
    EXPECT(test::throws([&] { make_op("unpack_int4").compute_shape({x}); }));
    EXPECT(make_op("convert", {{"target_type", shape::bf16_type}}).compute_shape({x}) ==
           shape{shape::bf16_type, {3, 4}});
}

TEST_CASE(view_shapes)
{
    shape x{shape::float_type, {3, 4}};
    EXPECT(make_op("transpose", {{"permutation", {1, 0}}}).compute_shape({x}) ==
           shape{shape::float_type, {4, 3}, {1, 4}});
    EXPECT(test::throws([&] { make_op("transpose", {{"permutation", {1, 1}}}).compute_shape({x}); }));
    shape v{shape::float_type, {4}};
    std::vector<std::size_t> lens = {3, 4};
    EXPECT(make_op("broadcast", {{"axis", 1}, {"out_lens", lens}}).compute_shape({v}) ==
           shape{shape::float_type, {3, 4}, {0, 1}});
    EXPECT(test::throws([&] { make_op("broadcast", {{"axis", 0}, {"out_lens", lens}}).compute_shape({v}); }));
    EXPECT(make_op("multibroadcast", {{"out_lens", lens}}).compute_shape({shape{shape::float_type}}) ==
           shape{shape::float_type, {3, 4}, {0, 0}});
    EXPECT(make_op("multibroadcast", {{"out_lens", lens}}).compute_shape({shape{shape::float_type, {3, 1}}}) ==
           shape{shape::float_type, {3, 4}, {1, 0}});
    EXPECT(make_op("reshape", {{"dims", {2, -1}}}).compute_shape({x}).lens() == std::vector<std::size_t>{2, 6});
    EXPECT(test::throws([&] { make_op("reshape", {{"dims", {5, -1}}}).compute_shape({x}); }));
    EXPECT(make_op("unsqueeze", {{"axes", {2}}}).compute_shape({x}) ==
           shape{shape::float_type, {3, 4, 1}, {4, 1, 1}});
    EXPECT(make_op("squeeze", {{"axes", {0}}}).compute_shape({shape{shape::float_type, {1, 4}}}).lens() ==
           std::vector<std::size_t>{4});
    auto sl = make_op("slice", {{"axes", {1}}, {"starts", {1}}, {"ends", {3}}});
    EXPECT(sl.compute_shape({x}) == shape{shape::float_type, {3, 2}, {4, 1}});
    argument a{x, std::vector<float>{0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11}};
    EXPECT(sl.compute(sl.compute_shape({x}), {a}).to_vector<float>() ==
           std::vector<float>{1, 2, 5, 6, 9, 10});
    auto tr = make_op("transpose", {{"permutation", {1, 0}}});
    auto at = tr.compute(tr.compute_shape({x}), {a});
    EXPECT(make_op("contiguous").compute(shape{shape::float_type, {4, 3}}, {at}).to_vector<float>() ==
           std::vector<float>{0, 4, 8, 1, 5, 9, 2, 6, 10, 3, 7, 11});
}

// ---------------------------------------------------------------- module, registries

TEST_CASE(module_editing)
{
    module m;
    auto x   = m.add_parameter("x", shape{shape::float_type, {2, 3}});
    auto y   = m.add_parameter("y", shape{shape::float_type, {2, 3}});
    auto l   = m.add_literal(literal{shape{shape::float_type, {2, 3}}, std::vector<float>{1, 2, 3, 4, 5, 6}});
    auto s   = m.add_instruction(make_op("add"), x, y);
    auto d   = m.add_instruction(make_op("mul"), x, l); // dead
    auto r   = m.add_instruction(make_op("sub"), s, y);
    (void)d;
    EXPECT(m.validate() == m.end());
    EXPECT(m.get_parameter_names() == std::vector<std::string>{"x", "y"});
    EXPECT(m.get_output_shapes().front() == shape{shape::float_type, {2, 3}});
    EXPECT(s->outputs().size() == 1 and x->outputs().size() == 2);
    migraphx::dead_code_elimination{}.apply(m);
    EXPECT(count_ops(m, "mul") == 0 and count_ops(m, "@literal") == 0 and count_ops(m, "@param") == 2);
    // replacing the last instruction keeps the replacement as the result
    auto t = m.insert_instruction(r, make_op("add"), s, s);
    m.replace_instruction(r, t);
    EXPECT(std::prev(m.end()) == t and m.validate() == m.end());
    // a shape change propagates to users
    module m2;
    auto p  = m2.add_parameter("p", shape{shape::float_type, {2, 3}});
    auto tp = m2.add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), p);
    auto id = m2.add_instruction(make_op("identity"), tp);
    m2.replace_instruction(tp, make_op("identity"), p);
    EXPECT(id->get_shape().lens() == std::vector<std::size_t>{2, 3});
    // copies are deep
    module m3 = m;
    EXPECT(m3 == m);
    m3.add_instruction(make_op("identity"), std::prev(m3.end()));
    EXPECT(m3 != m);
    auto tq = m2.add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), p);
    EXPECT(test::throws([&] { m2.add_instruction(make_op("add"), p, tq); }));
    EXPECT(test::throws([&] { m.remove_instruction(x); }));
}

TEST_CASE(registries)
{
    EXPECT(migraphx::has_op("quant_dot") and migraphx::has_op("unpack_int4") and
           migraphx::has_op("dequantizelinear") and migraphx::has_op("quantizelinear"));
    auto t = migraphx::make_target("oracle");
    EXPECT(t.name() == "oracle");
    bool thrown = false;
    try
    {
        migraphx::make_target("no_such_target");
    }
    catch(const migraphx::exception& e)
    {
        thrown = std::string(e.what()).find("Requested target 'no_such_target' is not loaded") !=
                 std::string::npos;
    }
    EXPECT(thrown);
    // an uncompiled arithmetic operator cannot be evaluated: there is no host fallback
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::int8_type, {2, 2}});
    mm->add_instruction(make_op("quant_dot"), x, x);
    argument a{shape{shape::int8_type, {2, 2}}, std::vector<int>{1, 2, 3, 4}};
    EXPECT(test::throws([&] { p.eval({{"x", a}}); }));
}

TEST_CASE(mi355_target_library_loads)
{
    // libmigraphx_mi355.so is found next to libmigraphx.so and registers the target and its
    // operators from its static initialisers; no GPU is touched by that
    auto t = migraphx::make_target("mi355");
    EXPECT(t.name() == "mi355");
    EXPECT(migraphx::has_op("mi355::quant_dot") and migraphx::has_op("mi355::w4a16_gemm"));
}

// ---------------------------------------------------------------- simplify_qdq

static void run_pass(module& m)
{
    migraphx::run_passes(m, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
}

// mul(broadcast s1, broadcast s2) as the pass emits it (test/simplify_qdq_test.cpp add_scale_mul)
static instruction_ref add_scale_mul(module& m,
                                     instruction_ref s1,
                                     instruction_ref s2,
                                     std::size_t axis1,
                                     std::size_t axis2,
                                     const std::vector<std::size_t>& out_lens)
{
    auto bc = [&](instruction_ref s, std::size_t axis) {
        if(s->get_shape().scalar())
            return m.add_instruction(make_op("multibroadcast", {{"out_lens", out_lens}}), s);
        return m.add_instruction(make_op("broadcast", {{"axis", axis}, {"out_lens", out_lens}}), s);
    };
    return m.add_instruction(make_op("mul"), bc(s1, axis1), bc(s2, axis2));
}

TEST_CASE(remove_qdq)
{
    shape sh{shape::float_type, {100, 100}};
    module m1;
    {
        auto t1    = m1.add_parameter("t1", sh);
        auto t2    = m1.add_parameter("t2", sh);
        auto scale = m1.add_literal(0.5f);
        auto zero  = m1.add_literal(std::int8_t{0});
        auto q1    = add_quantize_op(m1, "quantizelinear", t1, scale, zero);
        auto d1    = add_quantize_op(m1, "dequantizelinear", q1, scale, zero);
        auto q2    = add_quantize_op(m1, "quantizelinear", t2, scale, zero);
        auto d2    = add_quantize_op(m1, "dequantizelinear", q2, scale, zero);
        m1.add_return({m1.add_instruction(make_op("add"), d1, d2)});
    }
    module m2;
    {
        auto t1 = m2.add_parameter("t1", sh);
        auto t2 = m2.add_parameter("t2", sh);
        m2.add_return({m2.add_instruction(make_op("add"), t1, t2)});
    }
    run_pass(m1);
    EXPECT(canonical(m1) == canonical(m2));
}

TEST_CASE(qdq_different_scales)
{
    shape sh{shape::float_type, {100, 100}};
    module m1;
    {
        auto t1     = m1.add_parameter("t1", sh);
        auto scale1 = m1.add_literal(0.5f);
        auto scale2 = m1.add_literal(0.4f);
        auto zero   = m1.add_literal(std::int8_t{1});
        auto q1     = add_quantize_op(m1, "quantizelinear", t1, scale1, zero);
        auto d1     = add_quantize_op(m1, "dequantizelinear", q1, scale2, zero);
        m1.add_return({d1});
    }
    module m2 = m1;
    run_pass(m1);
    EXPECT(canonical(m1) == canonical(m2));
}

TEST_CASE(qdq_dot)
{
    // test/simplify_qdq_test.cpp:125-163
    shape sh1{shape::float_type, {1280, 1000}};
    shape sh2{shape::float_type, {1000, 1024}};
    module m1;
    {
        auto t1    = m1.add_parameter("t1", sh1);
        auto t2    = m1.add_parameter("t2", sh2);
        auto scale = m1.add_literal(0.5f);
        auto zero  = m1.add_literal(std::int8_t{0});
        auto q1    = add_quantize_op(m1, "quantizelinear", t1, scale, zero);
        auto d1    = add_quantize_op(m1, "dequantizelinear", q1, scale, zero);
        auto q2    = add_quantize_op(m1, "quantizelinear", t2, scale, zero);
        auto d2    = add_quantize_op(m1, "dequantizelinear", q2, scale, zero);
        m1.add_return({m1.add_instruction(make_op("dot"), d1, d2)});
    }
    module m3;
    {
        auto t1    = m3.add_parameter("t1", sh1);
        auto t2    = m3.add_parameter("t2", sh2);
        auto scale = m3.add_literal(0.5f);
        auto zero  = m3.add_literal(std::int8_t{0});
        auto q1    = add_quantize_op(m3, "quantizelinear", t1, scale, zero);
        auto q2    = add_quantize_op(m3, "quantizelinear", t2, scale, zero);
        auto dot   = m3.add_instruction(make_op("quant_dot"), q1, q2);
        auto os    = add_scale_mul(m3, scale, scale, 1, 1, dot->get_shape().lens());
        m3.add_return({m3.add_instruction(make_op("dequantizelinear"), dot, os)});
    }
    run_pass(m1);
    EXPECT(canonical(m1) == canonical(m3));
    EXPECT(count_ops(m1, "dot") == 0 and count_ops(m1, "quant_dot") == 1);
}

TEST_CASE(qdq_dot_fp16)
{
    // test/simplify_qdq_test.cpp:165-216: float Q/DQ parameters around a half dot
    shape sh1{shape::half_type, {64, 40}};
    shape sh2{shape::half_type, {40, 48}};
    module m1;
    {
        auto t1    = m1.add_parameter("t1", sh1);
        auto t2    = m1.add_parameter("t2", sh2);
        auto scale = m1.add_literal(0.5f);
        auto zero  = m1.add_literal(std::int8_t{0});
        auto c1 = m1.add_instruction(make_op("convert", {{"target_type", shape::float_type}}), t1);
        auto c2 = m1.add_instruction(make_op("convert", {{"target_type", shape::float_type}}), t2);
        auto q1 = add_quantize_op(m1, "quantizelinear", c1, scale, zero);
        auto d1 = add_quantize_op(m1, "dequantizelinear", q1, scale, zero);
        auto q2 = add_quantize_op(m1, "quantizelinear", c2, scale, zero);
        auto d2 = add_quantize_op(m1, "dequantizelinear", q2, scale, zero);
        auto h1 = m1.add_instruction(make_op("convert", {{"target_type", shape::half_type}}), d1);
        auto h2 = m1.add_instruction(make_op("convert", {{"target_type", shape::half_type}}), d2);
        m1.add_return({m1.add_instruction(make_op("dot"), h1, h2)});
    }
    run_pass(m1);
    EXPECT(count_ops(m1, "dot") == 0 and count_ops(m1, "quant_dot") == 1);
    auto last = m1.get_returns().front();
    EXPECT(last->name() == "convert" and last->get_shape().type() == shape::half_type);
    EXPECT(last->inputs().front()->name() == "dequantizelinear");
    EXPECT(last->inputs().front()->inputs().front()->get_shape().type() == shape::int32_type);
}

TEST_CASE(qdq_dot_multi_scale_and_transposed)
{
    // per-output-channel weight scale, weight stored [N, K] with the transpose between DQ and dot
    // (test/simplify_qdq_test.cpp:218-347)
    const std::size_t m = 16, k = 32, n = 24;
    module m1;
    {
        auto x   = m1.add_parameter("x", shape{shape::float_type, {m, k}});
        auto w   = m1.add_literal(literal{shape{shape::int8_type, {n, k}}, uniform_ints<int>(n * k, -127, 127, 3)});
        auto s1  = m1.add_literal(0.25f);
        auto z1  = m1.add_literal(std::int8_t{0});
        auto s2  = m1.add_literal(literal{shape{shape::float_type, {n}}, uniform_floats(n, 0.001f, 0.01f, 4)});
        auto z2  = m1.add_literal(literal{shape{shape::int8_type, {n}}, std::vector<int>(n, 0)});
        auto q1  = add_quantize_op(m1, "quantizelinear", x, s1, z1);
        auto d1  = add_quantize_op(m1, "dequantizelinear", q1, s1, z1);
        std::vector<std::size_t> wl = {n, k};
        auto s2b = m1.add_instruction(make_op("broadcast", {{"axis", 0}, {"out_lens", wl}}), s2);
        auto z2b = m1.add_instruction(make_op("broadcast", {{"axis", 0}, {"out_lens", wl}}), z2);
        auto d2  = m1.add_instruction(make_op("dequantizelinear"), w, s2b, z2b);
        auto wt  = m1.add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), d2);
        m1.add_return({m1.add_instruction(make_op("dot"), d1, wt)});
    }
    program before;
    *before.get_main_module() = m1;
    run_pass(m1);
    EXPECT(count_ops(m1, "dot") == 0 and count_ops(m1, "quant_dot") == 1);
    // the quantized weight reaches quant_dot through the re-applied transpose
    auto dq = m1.get_returns().front();
    EXPECT(dq->name() == "dequantizelinear" and dq->inputs().size() == 2);
    auto qd = dq->inputs()[0];
    EXPECT(qd->inputs()[1]->name() == "transpose" and qd->inputs()[1]->get_shape().type() == shape::int8_type);
    auto mul = dq->inputs()[1];
    EXPECT(mul->name() == "mul" and mul->inputs()[0]->name() == "multibroadcast" and
           mul->inputs()[1]->name() == "broadcast");
    EXPECT(migraphx::any_cast<migraphx::op::broadcast>(mul->inputs()[1]->get_operator()).axis == 1);
    // same numbers before and after, up to the float rounding of the fake-quantized dot
    program after;
    *after.get_main_module() = m1;
    argument xa{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 5)};
    auto r0 = run_on("oracle", before, {{"x", xa}});
    auto r1 = run_on("oracle", after, {{"x", xa}});
    EXPECT(max_rel_diff(r1[0], r0[0], 1.0) < 1e-5);
}

TEST_CASE(qdq_dot_unsupported_axis_and_uint8)
{
    // a per-row scale on the weight (length K on axis 0 of [K, N]) cannot move behind the dot
    // (test/simplify_qdq_test.cpp:445-477); uint8 tensors are left alone (:628-658)
    const std::size_t m = 8, k = 16, n = 12;
    module m1;
    {
        auto x  = m1.add_parameter("x", shape{shape::float_type, {m, k}});
        auto w  = m1.add_parameter("w", shape{shape::float_type, {k, n}});
        auto s1 = m1.add_literal(0.5f);
        auto z1 = m1.add_literal(std::int8_t{0});
        auto s2 = m1.add_literal(literal{shape{shape::float_type, {k}}, uniform_floats(k, 0.1f, 0.2f, 1)});
        auto z2 = m1.add_literal(literal{shape{shape::int8_type, {k}}, std::vector<int>(k, 0)});
        auto q1 = add_quantize_op(m1, "quantizelinear", x, s1, z1);
        auto d1 = add_quantize_op(m1, "dequantizelinear", q1, s1, z1);
        std::vector<std::size_t> wl = {k, n};
        auto s2b = m1.add_instruction(make_op("broadcast", {{"axis", 0}, {"out_lens", wl}}), s2);
        auto z2b = m1.add_instruction(make_op("broadcast", {{"axis", 0}, {"out_lens", wl}}), z2);
        auto q2  = m1.add_instruction(make_op("quantizelinear"), w, s2b, z2b);
        auto d2  = m1.add_instruction(make_op("dequantizelinear"), q2, s2b, z2b);
        m1.add_return({m1.add_instruction(make_op("dot"), d1, d2)});
    }
    run_pass(m1);
    EXPECT(count_ops(m1, "dot") == 1 and count_ops(m1, "quant_dot") == 0);

    module m2;
    {
        auto x  = m2.add_parameter("x", shape{shape::float_type, {m, k}});
        auto w  = m2.add_parameter("w", shape{shape::float_type, {k, n}});
        auto s  = m2.add_literal(0.5f);
        auto z  = m2.add_literal(std::uint8_t{0});
        auto q1 = add_quantize_op(m2, "quantizelinear", x, s, z);
        auto d1 = add_quantize_op(m2, "dequantizelinear", q1, s, z);
        auto q2 = add_quantize_op(m2, "quantizelinear", w, s, z);
        auto d2 = add_quantize_op(m2, "dequantizelinear", q2, s, z);
        m2.add_return({m2.add_instruction(make_op("dot"), d1, d2)});
    }
    run_pass(m2);
    // the fake-quantization pairs fold away, the dot stays a float dot
    EXPECT(count_ops(m2, "dot") == 1 and count_ops(m2, "quant_dot") == 0);
}

static module asymmetric_dot(int zp1, int zp2, std::size_t m, std::size_t k, std::size_t n)
{
    module m1;
    auto x  = m1.add_parameter("x", shape{shape::float_type, {m, k}});
    auto w  = m1.add_parameter("w", shape{shape::float_type, {k, n}});
    auto s1 = m1.add_literal(0.05f);
    auto s2 = m1.add_literal(0.02f);
    auto z1 = m1.add_literal(static_cast<std::int8_t>(zp1));
    auto z2 = m1.add_literal(static_cast<std::int8_t>(zp2));
    auto q1 = add_quantize_op(m1, "quantizelinear", x, s1, z1);
    auto d1 = add_quantize_op(m1, "dequantizelinear", q1, s1, z1);
    auto q2 = add_quantize_op(m1, "quantizelinear", w, s2, z2);
    auto d2 = add_quantize_op(m1, "dequantizelinear", q2, s2, z2);
    m1.add_return({m1.add_instruction(make_op("dot"), d1, d2)});
    return m1;
}

TEST_CASE(qdq_dot_asymmetric)
{
    // test/simplify_qdq_test.cpp:479-626 and :1471-1520: one extra quant_dot per non-zero zero
    // point, a third for the cross term, and the same numbers as the fake-quantized graph
    const std::size_t m = 12, k = 40, n = 20;
    struct cfg
    {
        int zp1, zp2;
        std::size_t quant_dots, adds, subs;
    };
    for(auto c : {cfg{3, 0, 2, 1, 0}, cfg{0, -5, 2, 1, 0}, cfg{3, -5, 4, 2, 1}, cfg{0, 0, 1, 0, 0}})
    {
        module m1 = asymmetric_dot(c.zp1, c.zp2, m, k, n);
        program before;
        *before.get_main_module() = m1;
        run_pass(m1);
        EXPECT(count_ops(m1, "dot") == 0);
        EXPECT(count_ops(m1, "quant_dot") == c.quant_dots);
        EXPECT(count_ops(m1, "add") == c.adds and count_ops(m1, "sub") == c.subs);
        auto dq = m1.get_returns().front();
        EXPECT(dq->inputs().size() == ((c.zp1 != 0 or c.zp2 != 0) ? 3u : 2u));
        program after;
        *after.get_main_module() = m1;
        argument xa{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 6)};
        argument wa{shape{shape::float_type, {k, n}}, normal_floats(k * n, 0.5f, 7)};
        auto r0 = run_on("oracle", before, {{"x", xa}, {"w", wa}});
        auto r1 = run_on("oracle", after, {{"x", xa}, {"w", wa}});
        EXPECT(max_rel_diff(r1[0], r0[0], 1e-2) < 1e-4);
    }
}

// ---------------------------------------------------------------- convolution

static migraphx::operation conv_op(const std::string& name,
                                   std::vector<int64_t> padding = {0, 0, 0, 0},
                                   std::vector<int64_t> stride  = {1, 1},
                                   std::vector<int64_t> dilation = {1, 1},
                                   int64_t group                = 1)
{
    return make_op(name, {{"padding", padding}, {"stride", stride}, {"dilation", dilation}, {"group", group},
                          {"padding_mode", 0}});
}

TEST_CASE(quant_convolution_shapes)
{
    // op/quant_convolution.hpp:85-134
    auto out = [](shape x, shape w, const migraphx::operation& op) { return op.compute_shape({x, w}); };
    EXPECT(out({shape::int8_type, {2, 3, 4, 4}}, {shape::int8_type, {2, 3, 3, 3}}, make_op("quant_convolution")) ==
           shape{shape::int32_type, {2, 2, 2, 2}});
    EXPECT(out({shape::int8_type, {2, 3, 4, 4}}, {shape::int8_type, {2, 3, 3, 3}},
               make_op("quant_convolution", {{"padding", {1, 1}}, {"stride", {2, 2}}})) ==
           shape{shape::int32_type, {2, 2, 2, 2}});
    EXPECT(out({shape::fp8e4m3fn_type, {1, 8, 9, 9}}, {shape::fp8e4m3fn_type, {4, 4, 3, 3}},
               conv_op("quant_convolution", {1, 1, 1, 1}, {1, 1}, {2, 2}, 2)) ==
           shape{shape::float_type, {1, 4, 7, 7}});
    // two padding entries per dimension: left ones first
    EXPECT(out({shape::int8_type, {1, 1, 5, 5}}, {shape::int8_type, {1, 1, 3, 3}},
               conv_op("quant_convolution", {0, 1, 2, 1})) == shape{shape::int32_type, {1, 1, 5, 5}});
    EXPECT(out({shape::float_type, {1, 4, 10}}, {shape::float_type, {6, 2, 3}},
               make_op("convolution", {{"padding", {1}}, {"stride", {2}}, {"dilation", {1}}, {"group", 2}})) ==
           shape{shape::float_type, {1, 6, 5}});
    // three spatial axes, the shapes of test/ref/convolution.cpp:859-1060 and one with every attribute
    EXPECT(out({shape::int8_type, {2, 3, 4, 4, 1}}, {shape::int8_type, {2, 3, 3, 3, 1}},
               make_op("quant_convolution", {{"padding", {0, 0, 0}}, {"stride", {1, 1, 1}}, {"dilation", {1, 1, 1}}})) ==
           shape{shape::int32_type, {2, 2, 2, 2, 1}});
    EXPECT(out({shape::int8_type, {1, 4, 9, 8, 7}}, {shape::int8_type, {6, 2, 3, 2, 3}},
               make_op("quant_convolution",
                       {{"padding", {1, 0, 2, 0, 1, 2}}, {"stride", {2, 1, 3}}, {"dilation", {1, 2, 1}}, {"group", 2}})) ==
           shape{shape::int32_type, {1, 6, 4, 7, 3}});
    EXPECT(test::throws([&] {
        out({shape::int8_type, {2, 3, 4, 4}}, {shape::int8_type, {2, 2, 3, 3}}, make_op("quant_convolution"));
    }));
    EXPECT(test::throws([&] {
        out({shape::uint8_type, {2, 3, 4, 4}}, {shape::uint8_type, {2, 3, 3, 3}}, make_op("quant_convolution"));
    }));
    EXPECT(test::throws([&] {
        out({shape::int8_type, {2, 3, 4, 4}}, {shape::int8_type, {2, 3, 3, 3}},
            make_op("quant_convolution", {{"stride", {1, 1, 1}}}));
    }));
}

TEST_CASE(quant_convolution_known_answers)
{
    // test/ref/quant_convolution.cpp:33-133 on the CPU target
    struct kat
    {
        std::vector<int64_t> padding, stride;
        std::vector<int> gold;
    };
    const std::vector<kat> cases = {
        {{0, 0}, {1, 1}, {10197, 10548, 11601, 11952, 25506, 26586, 29826, 30906, 27045, 27396, 28449, 28800,
                          77346, 78426, 81666, 82746}},
        {{1, 1}, {2, 2}, {4521, 7014, 7830, 11952, 10515, 16734, 19737, 30906, 13161, 19542, 19494, 28800,
                          34707, 52590, 54729, 82746}}};
    for(const auto& c : cases)
    {
        program p;
        auto* mm = p.get_main_module();
        std::vector<int> a(2 * 3 * 4 * 4), w(2 * 3 * 3 * 3);
        std::iota(a.begin(), a.end(), 0);
        std::iota(w.begin(), w.end(), 0);
        auto al = mm->add_literal(literal{shape{shape::int8_type, {2, 3, 4, 4}}, a});
        auto wl = mm->add_literal(literal{shape{shape::int8_type, {2, 3, 3, 3}}, w});
        mm->add_return({mm->add_instruction(
            make_op("quant_convolution", {{"padding", c.padding}, {"stride", c.stride}}), al, wl)});
        auto r = run_on("oracle", p, {});
        EXPECT(r[0].get_shape() == shape{shape::int32_type, {2, 2, 2, 2}});
        EXPECT(r[0].to_vector<int>() == c.gold);
    }
}

TEST_CASE(convolution_three_spatial_axes_on_cpu)
{
    // int8 operands over a volume on the CPU target against sums written out here: every output of
    // a 2 x 2 x 2 window over a 3 x 3 x 3 volume of ones times weights 1..8 is 36, a border of
    // zeros removes the weights that fall outside
    program p;
    auto* mm = p.get_main_module();
    std::vector<int> w(8);
    std::iota(w.begin(), w.end(), 1);
    auto x  = mm->add_literal(literal{shape{shape::int8_type, {1, 1, 3, 3, 3}}, std::vector<int>(27, 1)});
    auto wl = mm->add_literal(literal{shape{shape::int8_type, {1, 1, 2, 2, 2}}, w});
    auto plain = mm->add_instruction(
        make_op("quant_convolution", {{"padding", {0, 0, 0}}, {"stride", {1, 1, 1}}, {"dilation", {1, 1, 1}}}), x, wl);
    auto padded = mm->add_instruction(
        make_op("quant_convolution", {{"padding", {1, 0, 0}}, {"stride", {2, 1, 1}}, {"dilation", {1, 1, 1}}}), x, wl);
    mm->add_return({plain, padded});
    auto r = run_on("oracle", p, {});
    EXPECT(r[0].get_shape() == shape{shape::int32_type, {1, 1, 2, 2, 2}});
    EXPECT(r[0].to_vector<int>() == std::vector<int>(8, 36));
    // depth positions -1..0 (only the window's second plane, weights 5..8, sees data) and 1..2
    EXPECT(r[1].get_shape() == shape{shape::int32_type, {1, 1, 2, 2, 2}});
    EXPECT(r[1].to_vector<int>() == std::vector<int>{26, 26, 26, 26, 36, 36, 36, 36});
}

TEST_CASE(qdq_conv)
{
    // test/simplify_qdq_test.cpp:762-811 (`conv`) and :876-926 (`conv_multi_scale`)
    shape s4{shape::int8_type, {1280, 320, 1, 1}};
    shape s7{shape::float_type, {1, 320, 7, 7}};
    for(bool per_channel : {false, true})
    {
        auto weight_scale = [&](module& m) {
            if(per_channel)
                return m.add_literal(literal{shape{shape::float_type, {1280}}, uniform_floats(1280, 0.01f, 0.1f, 3)});
            return m.add_literal(0.5f);
        };
        module m1;
        {
            auto input   = m1.add_parameter("input", s7);
            auto weights = m1.add_parameter("weights", s4);
            auto wscale  = weight_scale(m1);
            auto scale   = m1.add_literal(0.5f);
            auto zero    = m1.add_literal(std::int8_t{0});
            instruction_ref d1;
            if(per_channel)
            {
                auto sb = m1.add_instruction(make_op("broadcast", {{"axis", 0}, {"out_lens", s4.lens()}}), wscale);
                auto zb = m1.add_instruction(make_op("multibroadcast", {{"out_lens", s4.lens()}}), zero);
                d1      = m1.add_instruction(make_op("dequantizelinear"), weights, sb, zb);
            }
            else
                d1 = add_quantize_op(m1, "dequantizelinear", weights, wscale, zero);
            auto q1 = add_quantize_op(m1, "quantizelinear", input, scale, zero);
            auto d5 = add_quantize_op(m1, "dequantizelinear", q1, scale, zero);
            m1.add_return({m1.add_instruction(conv_op("convolution"), d5, d1)});
        }
        module m2;
        {
            auto input   = m2.add_parameter("input", s7);
            auto weights = m2.add_parameter("weights", s4);
            auto wscale  = weight_scale(m2);
            auto scale   = m2.add_literal(0.5f);
            auto zero    = m2.add_literal(std::int8_t{0});
            auto q1      = add_quantize_op(m2, "quantizelinear", input, scale, zero);
            auto c1      = m2.add_instruction(conv_op("quant_convolution"), q1, weights);
            auto os      = add_scale_mul(m2, scale, wscale, 1, 1, c1->get_shape().lens());
            m2.add_return({m2.add_instruction(make_op("dequantizelinear"), c1, os)});
        }
        run_pass(m1);
        EXPECT(canonical(m1) == canonical(m2));
        EXPECT(count_ops(m1, "convolution") == 0 and count_ops(m1, "quant_convolution") == 1);
    }
    // a scale per input channel of the weights is no valid quantization axis (:928-975): untouched
    {
        module m1;
        auto input   = m1.add_parameter("input", s7);
        auto weights = m1.add_parameter("weights", s4);
        auto wscale  = m1.add_literal(literal{shape{shape::float_type, {320}}, uniform_floats(320, 0.01f, 0.1f, 4)});
        auto scale   = m1.add_literal(0.5f);
        auto zero    = m1.add_literal(std::int8_t{0});
        auto sb = m1.add_instruction(make_op("broadcast", {{"axis", 1}, {"out_lens", s4.lens()}}), wscale);
        auto zb = m1.add_instruction(make_op("multibroadcast", {{"out_lens", s4.lens()}}), zero);
        auto d1 = m1.add_instruction(make_op("dequantizelinear"), weights, sb, zb);
        auto q1 = add_quantize_op(m1, "quantizelinear", input, scale, zero);
        auto d5 = add_quantize_op(m1, "dequantizelinear", q1, scale, zero);
        m1.add_return({m1.add_instruction(conv_op("convolution"), d5, d1)});
        run_pass(m1);
        EXPECT(count_ops(m1, "convolution") == 1 and count_ops(m1, "quant_convolution") == 0);
    }
}

TEST_CASE(qdq_conv_asymmetric)
{
    // test/simplify_qdq_test.cpp:813-874 (`conv_asymmetric_input`): one more quant_convolution per
    // non-zero zero point, a third for the cross term; the rewritten graph computes what the
    // fake-quantized one does (padding included: the zero-point term sees the same zero border)
    struct cfg
    {
        int zp_in, zp_w;
        std::size_t convs, adds, subs;
    };
    shape sx{shape::float_type, {2, 4, 6, 6}};
    shape sw{shape::float_type, {6, 4, 3, 3}};
    for(auto c : {cfg{0, 0, 1, 0, 0}, cfg{1, 0, 2, 1, 0}, cfg{0, -2, 2, 1, 0}, cfg{3, -2, 4, 2, 1}})
    {
        module m1;
        {
            auto input   = m1.add_parameter("x", sx);
            auto weights = m1.add_parameter("w", sw);
            auto scale   = m1.add_literal(0.25f);
            auto wscale  = m1.add_literal(0.125f);
            auto zp_in   = m1.add_literal(static_cast<std::int8_t>(c.zp_in));
            auto zp_w    = m1.add_literal(static_cast<std::int8_t>(c.zp_w));
            auto qw = add_quantize_op(m1, "quantizelinear", weights, wscale, zp_w);
            auto dw = add_quantize_op(m1, "dequantizelinear", qw, wscale, zp_w);
            auto q1 = add_quantize_op(m1, "quantizelinear", input, scale, zp_in);
            auto d5 = add_quantize_op(m1, "dequantizelinear", q1, scale, zp_in);
            m1.add_return({m1.add_instruction(conv_op("convolution", {1, 1, 1, 1}, {2, 1}), d5, dw)});
        }
        program before;
        *before.get_main_module() = m1;
        run_pass(m1);
        EXPECT(count_ops(m1, "convolution") == 0);
        EXPECT(count_ops(m1, "quant_convolution") == c.convs);
        EXPECT(count_ops(m1, "add") == c.adds and count_ops(m1, "sub") == c.subs);
        program after;
        *after.get_main_module() = m1;
        argument xa{sx, normal_floats(sx.elements(), 2.0f, 21)};
        argument wa{sw, normal_floats(sw.elements(), 1.0f, 22)};
        auto r0 = run_on("oracle", before, {{"x", xa}, {"w", wa}});
        auto r1 = run_on("oracle", after, {{"x", xa}, {"w", wa}});
        EXPECT(r1[0].get_shape() == shape{shape::float_type, {2, 6, 3, 6}});
        EXPECT(max_rel_diff(r1[0], r0[0], 1e-2) < 1e-4);
    }
}

// ---------------------------------------------------------------- quantize_int4, quantize_int8

// ---------------------------------------------------------------- MX block quantization (fp4)

static void run_mx_pass(module& m)
{
    migraphx::simplify_qdq sq;
    sq.use_mx_quant = true;
    migraphx::run_passes(m, {sq, migraphx::dead_code_elimination{}});
}

TEST_CASE(fp4_shapes)
{
    // op/unpack_fp4.hpp:61-76, op/pack_fp4.hpp:64-80
    auto un = make_op("unpack_fp4");
    EXPECT(un.compute_shape({shape{shape::fp4x2_type, {1, 3, 6, 12}}}) ==
           shape{shape::fp8e4m3fn_type, {1, 3, 6, 24}});
    EXPECT(make_op("unpack_fp4", {{"axis", 1}}).compute_shape({shape{shape::fp4x2_type, {2, 1}}}) ==
           shape{shape::fp8e4m3fn_type, {2, 2}});
    EXPECT(test::throws([&] { un.compute_shape({shape{shape::uint8_type, {2, 2}}}); }));
    auto pk = make_op("pack_fp4", {{"axis", 1}});
    EXPECT(pk.compute_shape({shape{shape::float_type, {2, 2}}}) == shape{shape::fp4x2_type, {2, 1}});
    EXPECT(test::throws([&] { pk.compute_shape({shape{shape::float_type, {2, 3}}}); }));
    EXPECT(shape{shape::fp4x2_type, {4, 4}}.bytes() == 16);
    EXPECT(shape::parse_type("fp4x2_type") == shape::fp4x2_type);
}

TEST_CASE(fp4_pack_unpack_known_answers)
{
    // test/ref/pack_unpack_fp4.cpp:34-89
    program p;
    auto* mm = p.get_main_module();
    auto l0  = mm->add_literal(literal{shape{shape::float_type, {2, 2}}, std::vector<float>{-2.f, 3.4f, 3.5f, 0.f}});
    auto pk  = mm->add_instruction(make_op("pack_fp4", {{"axis", 1}}), l0);
    auto un  = mm->add_instruction(make_op("unpack_fp4", {{"axis", 1}}), pk);
    mm->add_return({pk, un});
    auto r = testutil::run_on("oracle", p, {});
    EXPECT(r.size() == 2);
    EXPECT(r[0].get_shape() == shape{shape::fp4x2_type, {2, 1}});
    EXPECT(static_cast<uint8_t>(r[0].data()[0]) == 0x5C and static_cast<uint8_t>(r[0].data()[1]) == 0x06);
    EXPECT(r[1].to_vector<float>() == std::vector<float>{-2.f, 3.f, 4.f, 0.f});
}

TEST_CASE(fp4x2_quant_dot_even)
{
    // test/simplify_qdq_test.cpp:1776-1814
    shape pa{shape::fp4x2_type, {1, 3, 6, 12}};
    shape pb{shape::fp4x2_type, {1, 3, 24, 4}};
    shape sa{shape::float_type, {1, 3, 6, 24}};
    shape sb{shape::float_type, {1, 3, 24, 8}};
    module m1;
    {
        auto a   = m1.add_parameter("input", pa);
        auto b   = m1.add_parameter("weights", pb);
        auto s1  = m1.add_parameter("scale_a", sa);
        auto s2  = m1.add_parameter("scale_b", sb);
        auto ua  = m1.add_instruction(make_op("unpack_fp4"), a);
        auto ub  = m1.add_instruction(make_op("unpack_fp4"), b);
        auto da  = m1.add_instruction(make_op("dequantizelinear"), ua, s1);
        auto db  = m1.add_instruction(make_op("dequantizelinear"), ub, s2);
        m1.add_return({m1.add_instruction(make_op("dot"), da, db)});
    }
    module m2;
    {
        auto a  = m2.add_parameter("input", pa);
        auto b  = m2.add_parameter("weights", pb);
        auto s1 = m2.add_parameter("scale_a", sa);
        auto s2 = m2.add_parameter("scale_b", sb);
        auto ua = m2.add_instruction(make_op("unpack_fp4"), a);
        auto ub = m2.add_instruction(make_op("unpack_fp4"), b);
        m2.add_return({m2.add_instruction(make_op("quant_dot"), ua, ub, s1, s2)});
    }
    run_mx_pass(m1);
    EXPECT(testutil::canonical(m1) == testutil::canonical(m2));
    // without the option the graph stays as it is
    module m3 = m2;
    run_pass(m3);
    EXPECT(testutil::canonical(m3) == testutil::canonical(m2));
}

TEST_CASE(fp4x2_quant_dot_trans_b)
{
    // test/simplify_qdq_test.cpp:1816-1860: the transpose between DQ and dot moves to the packed
    // tensor's unpacked form and to its scales
    shape pa{shape::fp4x2_type, {1, 3, 6, 12}};
    shape pb{shape::fp4x2_type, {1, 3, 8, 12}};
    shape sa{shape::float_type, {1, 3, 6, 24}};
    shape sb{shape::float_type, {1, 3, 8, 24}};
    module m1;
    {
        auto a  = m1.add_parameter("input", pa);
        auto b  = m1.add_parameter("weights", pb);
        auto s1 = m1.add_parameter("scale_a", sa);
        auto s2 = m1.add_parameter("scale_b", sb);
        auto ua = m1.add_instruction(make_op("unpack_fp4"), a);
        auto ub = m1.add_instruction(make_op("unpack_fp4"), b);
        auto da = m1.add_instruction(make_op("dequantizelinear"), ua, s1);
        auto db = m1.add_instruction(make_op("dequantizelinear"), ub, s2);
        auto tb = m1.add_instruction(make_op("transpose", {{"permutation", {0, 1, 3, 2}}}), db);
        m1.add_return({m1.add_instruction(make_op("dot"), da, tb)});
    }
    module m2;
    {
        auto a   = m2.add_parameter("input", pa);
        auto b   = m2.add_parameter("weights", pb);
        auto s1  = m2.add_parameter("scale_a", sa);
        auto s2  = m2.add_parameter("scale_b", sb);
        auto ua  = m2.add_instruction(make_op("unpack_fp4"), a);
        auto ub  = m2.add_instruction(make_op("unpack_fp4"), b);
        auto tb  = m2.add_instruction(make_op("transpose", {{"permutation", {0, 1, 3, 2}}}), ub);
        auto ts2 = m2.add_instruction(make_op("transpose", {{"permutation", {0, 1, 3, 2}}}), s2);
        m2.add_return({m2.add_instruction(make_op("quant_dot"), ua, tb, s1, ts2)});
    }
    run_mx_pass(m1);
    EXPECT(testutil::canonical(m1) == testutil::canonical(m2));
}

TEST_CASE(fp4x2_quant_dot_const_b)
{
    // test/simplify_qdq_test.cpp:1862-1905: constant packed weights and scales
    shape pa{shape::fp4x2_type, {1, 3, 6, 12}};
    shape pb{shape::fp4x2_type, {1, 3, 24, 4}};
    shape sa{shape::float_type, {1, 3, 6, 24}};
    shape sb{shape::float_type, {1, 3, 24, 8}};
    const auto bytes = testutil::uniform_ints<uint8_t>(pb.elements(), 0, 255, 826);
    const auto sbv   = testutil::uniform_floats(sb.elements(), 0.25f, 4.0f, 826);
    auto build = [&](module& m, bool rewritten) {
        auto a  = m.add_parameter("input", pa);
        auto b  = m.add_literal(literal{pb, reinterpret_cast<const char*>(bytes.data())});
        auto s1 = m.add_parameter("scale_a", sa);
        auto s2 = m.add_literal(literal{sb, sbv});
        auto ua = m.add_instruction(make_op("unpack_fp4"), a);
        auto ub = m.add_instruction(make_op("unpack_fp4"), b);
        if(rewritten)
        {
            m.add_return({m.add_instruction(make_op("quant_dot"), ua, ub, s1, s2)});
            return;
        }
        auto da = m.add_instruction(make_op("dequantizelinear"), ua, s1);
        auto db = m.add_instruction(make_op("dequantizelinear"), ub, s2);
        m.add_return({m.add_instruction(make_op("dot"), da, db)});
    };
    module m1;
    module m2;
    build(m1, false);
    build(m2, true);
    run_mx_pass(m1);
    EXPECT(testutil::canonical(m1) == testutil::canonical(m2));
}

TEST_CASE(mx_quant_dot_equals_dequantized_dot)
{
    // the rewritten graph computes what the fake-quantized one does: bit for bit on the CPU target,
    // because DQ of an fp8 value by a float scale is the same single float product
    const std::size_t m = 6, k = 64, n = 8;
    shape pa{shape::fp4x2_type, {m, k / 2}};
    shape pb{shape::fp4x2_type, {n, k / 2}};
    shape sa{shape::float_type, {m, k}};
    shape sb{shape::float_type, {n, k}};
    program p;
    {
        auto* mm = p.get_main_module();
        auto a   = mm->add_parameter("a", pa);
        auto b   = mm->add_parameter("b", pb);
        auto s1  = mm->add_parameter("sa", sa);
        auto s2  = mm->add_parameter("sb", sb);
        auto ua  = mm->add_instruction(make_op("unpack_fp4"), a);
        auto ub  = mm->add_instruction(make_op("unpack_fp4"), b);
        auto da  = mm->add_instruction(make_op("dequantizelinear"), ua, s1);
        auto db  = mm->add_instruction(make_op("dequantizelinear"), ub, s2);
        auto tb  = mm->add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), db);
        mm->add_return({mm->add_instruction(make_op("dot"), da, tb)});
    }
    program q = p;
    run_mx_pass(*q.get_main_module());
    EXPECT(testutil::count_ops(*q.get_main_module(), "quant_dot") == 1);
    EXPECT(testutil::count_ops(*q.get_main_module(), "dequantizelinear") == 0);
    argument aa{pa};
    argument ba{pb};
    const auto ca = testutil::uniform_ints<uint8_t>(pa.elements(), 0, 255, 1);
    const auto cb = testutil::uniform_ints<uint8_t>(pb.elements(), 0, 255, 2);
    std::memcpy(aa.data(), ca.data(), ca.size());
    std::memcpy(ba.data(), cb.data(), cb.size());
    auto block_scales = [](std::size_t rows, std::size_t kk, unsigned seed) {
        auto e = testutil::uniform_ints<int>(rows * (kk / 32), -4, 4, seed);
        std::vector<float> v(rows * kk);
        for(std::size_t i = 0; i < v.size(); i++)
            v[i] = std::ldexp(1.0f, e[i / 32]);
        return v;
    };
    migraphx::parameter_map params = {{"a", aa}, {"b", ba}, {"sa", argument{sa, block_scales(m, k, 3)}},
                                      {"sb", argument{sb, block_scales(n, k, 4)}}};
    auto want = testutil::run_on("oracle", p, params);
    auto got  = testutil::run_on("oracle", q, params);
    EXPECT(testutil::same_bytes(got[0], want[0]));
}

TEST_CASE(int4_pass)
{
    // test/int4_test.cpp:38-90
    const std::size_t m = 4, k = 6, n = 8;
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {m, k}});
    auto wv  = uniform_floats(k * n, -1.0f, 2.0f, 9);
    auto w   = mm->add_literal(literal{shape{shape::float_type, {k, n}}, wv});
    mm->add_return({mm->add_instruction(make_op("dot"), x, w)});
    program fp = p;
    migraphx::quantize_int4_weights(p);
    EXPECT(count_ops(*mm, "quantizelinear") == 1 and count_ops(*mm, "pack_int4") == 1 and
           count_ops(*mm, "unpack_int4") == 1 and count_ops(*mm, "dequantizelinear") == 1);
    auto dot = mm->get_returns().front();
    EXPECT(dot->name() == "dot" and dot->inputs()[0] == x);
    auto dq = dot->inputs()[1];
    EXPECT(dq->name() == "dequantizelinear" and dq->inputs()[0]->name() == "unpack_int4");
    auto q = dq->inputs()[0]->inputs()[0]->inputs()[0];
    EXPECT(q->name() == "quantizelinear" and q->get_shape().type() == shape::uint8_type);
    // per-tensor parameters: scale = (max - min) / 15, zero point = round(-min / scale)
    const float lo = std::min(0.0f, *std::min_element(wv.begin(), wv.end()));
    const float hi = std::max(0.0f, *std::max_element(wv.begin(), wv.end()));
    auto scale_lit = q->inputs()[1]->inputs()[0];
    auto zp_lit    = q->inputs()[2]->inputs()[0];
    EXPECT(scale_lit->get_literal().at<float>() == (hi - lo) / 15);
    EXPECT(zp_lit->get_literal().at<int>() == static_cast<int>(std::round(-lo / ((hi - lo) / 15))));
    // quantized weights stay within half a step of the originals
    argument xa{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 10)};
    auto r0 = run_on("oracle", fp, {{"x", xa}});
    auto r1 = run_on("oracle", p, {{"x", xa}});
    auto a  = r0[0].to_vector<double>();
    auto b  = r1[0].to_vector<double>();
    for(std::size_t i = 0; i < a.size(); i++)
        EXPECT(std::fabs(a[i] - b[i]) < 0.5 * (hi - lo) / 15 * k * 3);
    // an odd last dimension is left alone
    program p2;
    auto* m2 = p2.get_main_module();
    auto x2  = m2->add_parameter("x", shape{shape::float_type, {m, k}});
    auto w2  = m2->add_literal(literal{shape{shape::float_type, {k, 7}}, uniform_floats(k * 7, -1, 1, 1)});
    m2->add_return({m2->add_instruction(make_op("dot"), x2, w2)});
    migraphx::quantize_int4_weights(p2);
    EXPECT(count_ops(*m2, "quantizelinear") == 0);
}

TEST_CASE(int4_pass_takes_convolution_weights)
{
    // src/quantize_int4.cpp:40 lists convolution beside dot: constant weights with an even last
    // dimension go through the 4-bit store, the data input (a parameter) does not
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {1, 3, 8, 8}});
    auto wv  = uniform_floats(4 * 3 * 3 * 4, -0.5f, 1.0f, 19);
    auto w   = mm->add_literal(literal{shape{shape::float_type, {4, 3, 3, 4}}, wv});
    mm->add_return({mm->add_instruction(make_op("convolution"), x, w)});
    program fp = p;
    migraphx::quantize_int4_weights(p);
    EXPECT(count_ops(*mm, "quantizelinear") == 1 and count_ops(*mm, "pack_int4") == 1 and
           count_ops(*mm, "unpack_int4") == 1 and count_ops(*mm, "dequantizelinear") == 1);
    auto conv = mm->get_returns().front();
    EXPECT(conv->name() == "convolution" and conv->inputs()[0] == x);
    EXPECT(conv->inputs()[1]->name() == "dequantizelinear");
    EXPECT(conv->get_shape() == fp.get_main_module()->get_returns().front()->get_shape());
    // 3 x 3 windows: the odd last dimension stays in float
    program p2;
    auto* m2 = p2.get_main_module();
    auto x2  = m2->add_parameter("x", shape{shape::float_type, {1, 3, 8, 8}});
    auto w2  = m2->add_literal(literal{shape{shape::float_type, {4, 3, 3, 3}}, uniform_floats(108, -1, 1, 2)});
    m2->add_return({m2->add_instruction(make_op("convolution"), x2, w2)});
    migraphx::quantize_int4_weights(p2);
    EXPECT(count_ops(*m2, "quantizelinear") == 0);
}

TEST_CASE(int8_calibration)
{
    // test/quantization.cpp:1066-1110: calibrated int8 dot stays close to the float dot
    const std::size_t m = 16, k = 64, n = 32;
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {m, k}});
    auto wv  = normal_floats(k * n, 0.05f, 11);
    auto w   = mm->add_literal(literal{shape{shape::float_type, {k, n}}, wv});
    mm->add_return({mm->add_instruction(make_op("dot"), x, w)});
    program fp = p;
    auto xv    = normal_floats(m * k, 1.0f, 12);
    argument xa{shape{shape::float_type, {m, k}}, xv};
    migraphx::quantize_int8(p, migraphx::make_target("oracle"), {{{"x", xa}}});
    EXPECT(count_ops(*mm, "capture") == 0);
    EXPECT(count_ops(*mm, "quantizelinear") == 2 and count_ops(*mm, "dequantizelinear") == 2);
    // Q scale literal = max|x| / 127 (the inverse of the calibrated multiplier)
    float amax = 0;
    for(float v : xv)
        amax = std::max(amax, std::fabs(v));
    auto dot = mm->get_returns().front();
    auto dq  = dot->inputs()[0];
    auto sc  = dq->inputs()[1]->inputs()[0]->get_literal().at<float>();
    EXPECT(sc == 1.0f / (127.0f / amax));
    EXPECT(dq->inputs()[2]->get_shape().type() == shape::int8_type);
    EXPECT(test::throws([&] {
        program q = fp;
        migraphx::quantize_int8(q, migraphx::make_target("oracle"), {}, {"dot"});
    }));
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    EXPECT(count_ops(*mm, "quant_dot") == 1 and count_ops(*mm, "dot") == 0);
    auto r0 = run_on("oracle", fp, {{"x", xa}});
    auto r1 = run_on("oracle", p, {{"x", xa}});
    // root-mean-square error relative to the result's own RMS, as verify::rms_range compares
    auto a = r0[0].to_vector<double>();
    auto b = r1[0].to_vector<double>();
    double num = 0, den = 0;
    for(std::size_t i = 0; i < a.size(); i++)
    {
        num += (a[i] - b[i]) * (a[i] - b[i]);
        den += a[i] * a[i];
    }
    EXPECT(std::sqrt(num / den) < 0.02);
}

TEST_CASE(fp8_calibration)
{
    const std::size_t m = 8, k = 32, n = 16;
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {m, k}});
    auto w   = mm->add_literal(literal{shape{shape::float_type, {k, n}}, normal_floats(k * n, 0.02f, 13)});
    mm->add_return({mm->add_instruction(make_op("dot"), x, w)});
    program fp = p;
    argument xa{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 14)};
    migraphx::quantize_fp8(p, migraphx::make_target("oracle"), {{{"x", xa}}});
    auto dot = mm->get_returns().front();
    EXPECT(dot->inputs()[0]->inputs()[0]->get_shape().type() == shape::fp8e4m3fn_type);
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    EXPECT(count_ops(*mm, "quant_dot") == 1);
    EXPECT(mm->get_returns().front()->inputs()[0]->get_shape().type() == shape::float_type);
    auto r0 = run_on("oracle", fp, {{"x", xa}});
    auto r1 = run_on("oracle", p, {{"x", xa}});
    auto a  = r0[0].to_vector<double>();
    auto b  = r1[0].to_vector<double>();
    double num = 0, den = 0;
    for(std::size_t i = 0; i < a.size(); i++)
    {
        num += (a[i] - b[i]) * (a[i] - b[i]);
        den += a[i] * a[i];
    }
    EXPECT(std::sqrt(num / den) < 0.06);
}

// ---------------------------------------------------------------- encoder graph

TEST_CASE(encoder_graph_on_cpu)
{
    // the BERT-shaped graph of benchmark config 5, small: calibration, QDQ rewrite and evaluation on
    // the CPU oracle target; the int8 model must stay close to the float one
    encoder::config c;
    c.layers = 1;
    auto w   = encoder::make_weights(c, 3);
    argument ids{shape{shape::int32_type, {c.tokens()}}, uniform_ints<int>(c.tokens(), 0, static_cast<int>(c.vocab) - 1, 4)};
    auto scales = encoder::calibrate(c, w, "oracle", ids);
    EXPECT(scales.size() == 4);
    for(float s : scales)
        EXPECT(s > 0 and std::isfinite(s));
    auto p = encoder::quantized(c, w, scales);
    EXPECT(count_ops(*p.get_main_module(), "dot") == 8);
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    EXPECT(count_ops(*p.get_main_module(), "quant_dot") == 6);
    EXPECT(count_ops(*p.get_main_module(), "dot") == 2);
    EXPECT(count_ops(*p.get_main_module(), "quantizelinear") == 4);
    EXPECT(count_ops(*p.get_main_module(), "dequantizelinear") == 6);
    auto q = run_on("oracle", p, {{"ids", ids}});
    encoder::builder fb{c, w, {}, {}};
    fb.tap  = [](std::size_t, std::vector<argument>) {};
    auto fp = fb.build();
    auto f  = run_on("oracle", fp, {{"ids", ids}});
    auto a = q[0].to_vector<double>();
    auto b = f[0].to_vector<double>();
    double num = 0, den = 0;
    for(std::size_t i = 0; i < a.size(); i++)
    {
        EXPECT(std::isfinite(a[i]));
        num += (a[i] - b[i]) * (a[i] - b[i]);
        den += b[i] * b[i];
    }
    EXPECT(std::sqrt(num / den) < 0.05);
    // LayerNorm output: rows have mean ~beta and unit-scale spread
    EXPECT(q[0].get_shape() == shape{shape::float_type, {c.tokens(), c.hidden}});
}

// ---------------------------------------------------------------- saved programs
// Follows test/msgpack.cpp (encodings compared with the MessagePack format's own byte layouts),
// test/json.cpp and test/serialize_program.cpp (a program equals the one read back from its value,
// MessagePack, JSON and file forms, compiled or not).

static std::vector<char> bytes_of(std::initializer_list<int> b)
{
    std::vector<char> r;
    for(int x : b)
        r.push_back(static_cast<char>(x));
    return r;
}

TEST_CASE(msgpack_known_encodings)
{
    using migraphx::to_msgpack;
    using migraphx::value;
    // the MessagePack specification's formats: fixint, uint8/16/32/64, negative fixint, int8/16/32
    EXPECT(to_msgpack(value{}) == bytes_of({0xc0}));
    EXPECT(to_msgpack(value(true)) == bytes_of({0xc3}));
    EXPECT(to_msgpack(value(false)) == bytes_of({0xc2}));
    EXPECT(to_msgpack(value(3)) == bytes_of({0x03}));
    EXPECT(to_msgpack(value(127)) == bytes_of({0x7f}));
    EXPECT(to_msgpack(value(128)) == bytes_of({0xcc, 0x80}));
    EXPECT(to_msgpack(value(256)) == bytes_of({0xcd, 0x01, 0x00}));
    EXPECT(to_msgpack(value(65536)) == bytes_of({0xce, 0x00, 0x01, 0x00, 0x00}));
    EXPECT(to_msgpack(value(int64_t{1} << 32)) ==
           bytes_of({0xcf, 0, 0, 0, 1, 0, 0, 0, 0}));
    EXPECT(to_msgpack(value(-1)) == bytes_of({0xff}));
    EXPECT(to_msgpack(value(-32)) == bytes_of({0xe0}));
    EXPECT(to_msgpack(value(-33)) == bytes_of({0xd0, 0xdf}));
    EXPECT(to_msgpack(value(-129)) == bytes_of({0xd1, 0xff, 0x7f}));
    EXPECT(to_msgpack(value(-32769)) == bytes_of({0xd2, 0xff, 0xff, 0x7f, 0xff}));
    EXPECT(to_msgpack(value(-(int64_t{1} << 40))) ==
           bytes_of({0xd3, 0xff, 0xff, 0xff, 0, 0, 0, 0, 0}));
    // doubles are float64, big endian: 1.5 = 0x3ff8000000000000
    EXPECT(to_msgpack(value(1.5)) == bytes_of({0xcb, 0x3f, 0xf8, 0, 0, 0, 0, 0, 0}));
    EXPECT(to_msgpack(value("abc")) == bytes_of({0xa3, 'a', 'b', 'c'}));
    {
        const std::string s40(40, 'x');
        auto b = to_msgpack(value(s40));
        EXPECT(b.size() == 42 and static_cast<unsigned char>(b[0]) == 0xd9 and b[1] == 40);
    }
    EXPECT(to_msgpack(value(std::vector<int>{1, 2, 3})) == bytes_of({0x93, 1, 2, 3}));
    EXPECT(to_msgpack(value::array()) == bytes_of({0x90}));
    // keyed items make a map, in order
    EXPECT(to_msgpack(value{{"a", 1}, {"b", true}}) ==
           bytes_of({0x82, 0xa1, 'a', 0x01, 0xa1, 'b', 0xc3}));
    // binary data: an array of bin chunks (one here)
    const unsigned char raw[3] = {0, 200, 7};
    EXPECT(to_msgpack(value::binary(raw, 3)) == bytes_of({0x91, 0xc4, 3, 0, 200, 7}));
    {
        std::vector<int> many(20, 5);
        auto b = to_msgpack(value(many));
        EXPECT(static_cast<unsigned char>(b[0]) == 0xdc and b[1] == 0 and b[2] == 20 and b.size() == 23);
    }
}

TEST_CASE(msgpack_reads_every_number_format)
{
    using migraphx::from_msgpack;
    EXPECT(from_msgpack(bytes_of({0xca, 0x3f, 0xc0, 0, 0})).to<double>() == 1.5); // float32
    EXPECT(from_msgpack(bytes_of({0xcc, 0xff})).to<int>() == 255);
    EXPECT(from_msgpack(bytes_of({0xd0, 0x80})).to<int>() == -128);
    EXPECT(from_msgpack(bytes_of({0xd1, 0x80, 0x00})).to<int>() == -32768);
    EXPECT(from_msgpack(bytes_of({0xd2, 0x80, 0, 0, 0})).to<int64_t>() == -2147483648ll);
    EXPECT(from_msgpack(bytes_of({0xd3, 0xff, 0xff, 0xff, 0xff, 0xff, 0xff, 0xff, 0xfe})).to<int>() == -2);
    EXPECT(from_msgpack(bytes_of({0xda, 0, 2, 'h', 'i'})).to<std::string>() == "hi");
    EXPECT(from_msgpack(bytes_of({0xdd, 0, 0, 0, 2, 1, 2})).to_vector<int>() == std::vector<int>{1, 2});
    EXPECT(from_msgpack(bytes_of({0xde, 0, 1, 0xa1, 'k', 0x05})).at("k").to<int>() == 5);
    // a lone bin object (the older layout) and chunked binary both read as binary
    EXPECT(from_msgpack(bytes_of({0xc4, 2, 9, 8})).get_binary() == std::string("\x09\x08"));
    EXPECT(from_msgpack(bytes_of({0x92, 0xc4, 1, 9, 0xc5, 0, 1, 8})).get_binary() == std::string("\x09\x08"));
    // unsigned 64-bit: up to the signed range; above it the reader refuses instead of wrapping negative
    EXPECT(from_msgpack(bytes_of({0xcf, 0x7f, 0xff, 0xff, 0xff, 0xff, 0xff, 0xff, 0xff})).to<int64_t>() == INT64_MAX);
    EXPECT(test::throws([] { from_msgpack(bytes_of({0xcf, 0x80, 0, 0, 0, 0, 0, 0, 0})); }));
    EXPECT(test::throws([] { from_msgpack(bytes_of({0xc7, 1, 1, 0})); }));       // ext
    EXPECT(test::throws([] { from_msgpack(bytes_of({0xa5, 'a', 'b'})); }));      // truncated
    EXPECT(test::throws([] { from_msgpack(bytes_of({0x93, 1, 2})); }));          // truncated array
    EXPECT(test::throws([] { from_msgpack(std::vector<char>{}); }));
}

static migraphx::value sample_value()
{
    using migraphx::value;
    const unsigned char raw[5] = {1, 0, 255, 128, 3};
    value v                    = value::object();
    v["none"]                  = value("none", value{});
    v["flag"]                  = value("flag", true);
    v["count"]                 = value("count", -70000);
    v["big"]                   = value("big", int64_t{1} << 50);
    v["ratio"]                 = value("ratio", 0.1);
    v["whole"]                 = value("whole", 2.0);
    v["text"]                  = value("text", "line\n\"quoted\"\t\\ \x01 caf\xc3\xa9");
    v["list"]                  = value("list", std::vector<int>{1, -2, 3});
    v["empty"]                 = value("empty", value::array());
    v["bytes"]                 = value("bytes", value::binary(raw, 5));
    value inner                = value::object();
    inner["lens"]              = value("lens", std::vector<std::size_t>{2, 3});
    inner["nested"]            = value("nested", value{{"k", 1.25}});
    v["inner"]                 = value("inner", inner);
    return v;
}

TEST_CASE(msgpack_and_json_round_trips)
{
    auto v = sample_value();
    auto m = migraphx::from_msgpack(migraphx::to_msgpack(v));
    EXPECT(m == v);
    EXPECT(m.at("bytes").is_binary() and m.at("bytes").get_binary().size() == 5);
    EXPECT(m.at("whole").kind() == migraphx::value::float_kind);
    auto text = migraphx::to_json_string(v);
    auto j    = migraphx::from_json_string(text);
    EXPECT(j == v);
    EXPECT(j.at("whole").kind() == migraphx::value::float_kind);
    EXPECT(j.at("text").to<std::string>() == v.at("text").to<std::string>());
    // hand-written JSON: whitespace, escapes, exponents, nesting
    auto h = migraphx::from_json_string(
        " { \"a\" : [ 1 , 2.5e1 , -3 ] , \"s\" : \"\\u0041\\u00e9\\ud83d\\ude00\\/\" , \"o\" : { } , \"n\" : null }");
    EXPECT(h.at("a").to_vector<double>() == std::vector<double>{1, 25, -3});
    EXPECT(h.at("s").to<std::string>() == "A\xc3\xa9\xf0\x9f\x98\x80/");
    EXPECT(h.at("o").is_object() and h.at("o").empty());
    EXPECT(h.at("n").is_null());
    EXPECT(migraphx::to_json_string(migraphx::value{{"a", 1}, {"b", "x"}}) == "{\"a\":1,\"b\":\"x\"}");
    EXPECT(migraphx::to_json_string(migraphx::value(std::vector<int>{1, 2})) == "[1,2]");
    EXPECT(test::throws([] { migraphx::from_json_string("{\"a\": }"); }));
    EXPECT(test::throws([] { migraphx::from_json_string("[1, 2"); }));
    EXPECT(test::throws([] { migraphx::from_json_string("[1] x"); }));
}

TEST_CASE(shape_and_literal_values)
{
    shape s{shape::half_type, {2, 3, 4}, {12, 1, 3}};
    auto v = migraphx::to_value(s);
    EXPECT(v.at("type").to<std::string>() == "half_type");
    EXPECT(v.at("lens").to_vector<std::size_t>() == s.lens());
    EXPECT(v.at("strides").to_vector<std::size_t>() == s.strides());
    EXPECT(v.at("dynamic_dimensions").empty() and v.at("sub_shapes").empty());
    EXPECT(migraphx::from_value<shape>(v) == s);
    literal l{shape{shape::int8_type, {2, 2}}, std::vector<int>{-128, 127, 0, 5}};
    auto lv = migraphx::to_value(l);
    EXPECT(lv.at("data").get_binary() == std::string("\x80\x7f\x00\x05", 4));
    EXPECT(migraphx::from_value<literal>(lv) == l);
    // a literal whose byte count disagrees with its shape is refused
    lv["data"] = migraphx::value("data", migraphx::value::binary("ab", 2));
    EXPECT(test::throws([&] { migraphx::from_value<literal>(lv); }));
    // a scalar
    literal one{1.5f};
    EXPECT(migraphx::from_value<literal>(migraphx::to_value(one)) == one);
}

static program qdq_program_for_saving()
{
    // three parameters added in order, literals of several types, operators with list, number,
    // type and string attributes, views, and the quantize / dequantize pair
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {2, 4, 8}});
    auto w   = mm->add_parameter("w", shape{shape::float_type, {8, 6}});
    auto b   = mm->add_parameter("bias", shape{shape::half_type, {6}});
    auto sc  = mm->add_literal(literal{0.05f});
    auto zp  = mm->add_literal(literal{shape{shape::int8_type}, std::vector<int>{3}});
    auto qx  = add_quantize_op(*mm, "quantizelinear", x, sc, zp);
    auto dx  = add_quantize_op(*mm, "dequantizelinear", qx, sc, zp);
    auto wt  = mm->add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), w);
    auto wtt = mm->add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), wt);
    auto wb  = mm->add_instruction(make_op("multibroadcast", {{"out_lens", {2, 8, 6}}}), wtt);
    auto d   = mm->add_instruction(make_op("dot"), dx, wb);
    auto bf  = mm->add_instruction(make_op("convert", {{"target_type", shape::float_type}}), b);
    auto bb  = mm->add_instruction(make_op("multibroadcast", {{"out_lens", {2, 4, 6}}}), bf);
    auto sum = mm->add_instruction(make_op("add"), d, bb);
    auto sl  = mm->add_instruction(
        make_op("slice", {{"axes", {2}}, {"starts", {1}}, {"ends", {5}}}), sum);
    auto sm = mm->add_instruction(make_op("softmax", {{"axis", -1}}), sl);
    mm->add_return({sm, sum});
    return p;
}

static std::string printed(const program& p)
{
    std::stringstream ss;
    ss << p;
    return ss.str();
}

TEST_CASE(program_value_round_trip)
{
    auto p1 = qdq_program_for_saving();
    auto v  = p1.to_value();
    EXPECT(v.at("version").to<int>() == 8);
    EXPECT(v.at("targets").empty() and v.at("contexts").empty());
    const auto& nodes = v.at("modules").at("main").at("nodes");
    EXPECT(nodes.size() == p1.get_main_module()->size());
    // results are named by position, parameters by name; inputs refer to those names
    std::size_t i = 0;
    for(const auto& node : nodes.items())
    {
        const auto name = node.at("name").to<std::string>();
        if(name == "@param")
            EXPECT(node.at("output").to<std::string>() == node.at("operator").at("parameter").to<std::string>());
        else
            EXPECT(node.at("output").to<std::string>() == "@" + std::to_string(i));
        EXPECT(node.contains("literal") == (name == "@literal"));
        i++;
    }
    program p2;
    p2.from_value(v);
    EXPECT(p1 == p2);
    EXPECT(printed(p1) == printed(p2));
    EXPECT(p2.get_parameter_names() == p1.get_parameter_names());
    EXPECT(p2.get_output_shapes() == p1.get_output_shapes());
    EXPECT(not p2.is_compiled());
    EXPECT(p2.to_value() == v);
}

TEST_CASE(program_saved_as_msgpack_json_and_file)
{
    auto p1 = qdq_program_for_saving();
    for(const std::string format : {"msgpack", "json"})
    {
        migraphx::file_options o;
        o.format    = format;
        auto buffer = migraphx::save_buffer(p1, o);
        auto p2     = migraphx::load_buffer(buffer, o);
        EXPECT(p1 == p2);
        EXPECT(printed(p1) == printed(p2));
        auto p3 = migraphx::load_buffer(buffer.data(), buffer.size(), o);
        EXPECT(p1 == p3);
    }
    const std::string filename = "/tmp/mi355_host_tests_program.mxr";
    migraphx::save(p1, filename);
    auto p4 = migraphx::load(filename);
    std::remove(filename.c_str());
    EXPECT(p1 == p4);
    EXPECT(test::throws([&] { migraphx::load(filename); })); // gone
    migraphx::file_options bad;
    bad.format = "???";
    EXPECT(test::throws([&] { migraphx::save_buffer(p1, bad); }));
    EXPECT(test::throws([&] { migraphx::load_buffer(std::vector<char>{}, bad); }));
}

TEST_CASE(program_load_rejects_bad_files)
{
    auto v = qdq_program_for_saving().to_value();
    {
        auto w       = v;
        w["version"] = migraphx::value("version", 7);
        program p;
        EXPECT(test::throws([&] { p.from_value(w); }));
    }
    {
        // an input that is not defined yet
        program p;
        auto* mm = p.get_main_module();
        auto x   = mm->add_parameter("x", shape{shape::float_type, {2}});
        mm->add_instruction(make_op("neg"), x);
        auto text = migraphx::to_json_string(p.to_value());
        auto at   = text.find("\"inputs\":[\"x\"]");
        EXPECT(at != std::string::npos);
        text.replace(at, 14, "\"inputs\":[\"y\"]");
        migraphx::file_options o;
        o.format = "json";
        EXPECT(test::throws([&] { migraphx::load_buffer(text.data(), text.size(), o); }));
    }
    {
        // an operator this library does not have
        auto text = migraphx::to_json_string(v);
        auto at   = text.find("\"name\":\"softmax\"");
        EXPECT(at != std::string::npos);
        text.replace(at, 16, "\"name\":\"softmin\"");
        migraphx::file_options o;
        o.format = "json";
        EXPECT(test::throws([&] { migraphx::load_buffer(text.data(), text.size(), o); }));
    }
    // cut short
    auto buffer = migraphx::save_buffer(qdq_program_for_saving());
    buffer.resize(buffer.size() / 2);
    EXPECT(test::throws([&] { migraphx::load_buffer(buffer); }));
}

TEST_CASE(saved_program_evaluates_the_same)
{
    // the quantized form of a program (after the QDQ rewrite) is saved, read back, and both are
    // evaluated on the CPU oracle target; compiled there, it is saved and read back once more
    auto p1 = qdq_program_for_saving();
    migraphx::run_passes(p1, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    auto p2 = migraphx::load_buffer(migraphx::save_buffer(p1));
    EXPECT(p1 == p2);
    migraphx::parameter_map params;
    params["x"]    = argument{shape{shape::float_type, {2, 4, 8}}, normal_floats(64, 1.0f, 1)};
    params["w"]    = argument{shape{shape::float_type, {8, 6}}, normal_floats(48, 0.5f, 2)};
    params["bias"] = argument{shape{shape::half_type, {6}}, normal_floats(6, 0.5f, 3)};
    auto r1 = run_on("oracle", p1, params);
    auto r2 = run_on("oracle", p2, params);
    EXPECT(r1.size() == 2 and r2.size() == 2);
    EXPECT(same_bytes(r1[0], r2[0]) and same_bytes(r1[1], r2[1]));

    program c1 = p1;
    c1.compile(migraphx::make_target("oracle"));
    auto v = c1.to_value();
    EXPECT(v.at("targets").size() == 1);
    EXPECT(v.at("targets").at(0).at("name").to<std::string>() == "oracle");
    EXPECT(v.at("contexts").size() == 1);
    auto c2 = migraphx::load_buffer(migraphx::save_buffer(c1));
    EXPECT(c2.is_compiled());
    EXPECT(c1 == c2);
    auto r3 = c2.eval(params);
    c2.finish();
    EXPECT(same_bytes(r1[0], r3[0]) and same_bytes(r1[1], r3[1]));
    // a compiled program cannot be compiled again, loaded or not
    EXPECT(test::throws([&] { c2.compile(migraphx::make_target("oracle")); }));
}

// ---------------------------------------------------------------- MatMulNBits

TEST_CASE(matmulnbits_graph_checks)
{
    module m;
    auto a  = m.add_parameter("a", shape{shape::float_type, {2, 32}});
    auto b  = m.add_parameter("b", shape{shape::uint8_type, {4, 2, 8}});
    auto s  = m.add_parameter("s", shape{shape::float_type, {8}});
    auto r  = migraphx::op::builder::matmulnbits(m, a, b, s, m.end(), 4, 32, 16);
    EXPECT(r->get_shape() == shape{shape::float_type, {2, 4}});
    EXPECT(count_ops(m, "unpack_int4") == 1 and count_ops(m, "dequantizelinear") == 1);
    EXPECT(test::throws([&] { migraphx::op::builder::matmulnbits(m, a, b, s, m.end(), 4, 32, 24); }));
    EXPECT(test::throws([&] { migraphx::op::builder::matmulnbits(m, a, b, s, m.end(), 5, 32, 16); }));
    EXPECT(test::throws([&] { migraphx::op::builder::matmulnbits(m, a, b, a, m.end(), 4, 32, 16); }));
}

// `host_tests matmulnbits <target> <case file> <result file>`: build the MatMulNBits graph from a
// text description and evaluate it.  The Python tests feed it the reference's known answers.
static int matmulnbits_tool(int argc, char** argv)
{
    if(argc != 5)
        return 2;
    std::ifstream in(argv[3]);
    std::size_t nda = 0, n = 0, nblk = 0, blob = 0;
    int has_zp = 0, use_half = 0;
    in >> nda;
    std::vector<std::size_t> a_lens(nda);
    for(auto& l : a_lens)
        in >> l;
    in >> n >> nblk >> blob >> has_zp >> use_half;
    const std::size_t k   = a_lens.back();
    const std::size_t blk = blob * 2;
    std::size_t na        = 1;
    for(auto l : a_lens)
        na *= l;
    std::vector<float> a(na), scales(n * nblk);
    std::vector<int> b(n * nblk * blob), zp(has_zp != 0 ? n * ((nblk + 1) / 2) : 0);
    for(auto& v : a)
        in >> v;
    for(auto& v : b)
        in >> v;
    for(auto& v : scales)
        in >> v;
    for(auto& v : zp)
        in >> v;
    if(not in)
        return 3;
    const auto ft = use_half != 0 ? shape::half_type : shape::float_type;
    program p;
    auto* mm = p.get_main_module();
    auto ai  = mm->add_parameter("a", shape{ft, a_lens});
    auto bi  = mm->add_literal(literal{shape{shape::uint8_type, {n, nblk, blob}}, b});
    auto si  = mm->add_literal(literal{shape{ft, {n * nblk}}, scales});
    auto zi  = mm->end();
    if(has_zp != 0)
        zi = mm->add_literal(literal{shape{shape::uint8_type, {zp.size()}}, zp});
    mm->add_return({migraphx::op::builder::matmulnbits(*mm, ai, bi, si, zi, n, k, blk)});
    argument aa{shape{ft, a_lens}, a};
    auto r = run_on(argv[2], p, {{"a", aa}});
    std::ofstream out(argv[4]);
    out.precision(9);
    for(auto v : r[0].to_vector<float>())
        out << v << "\n";
    return 0;
}

// `host_tests onnx print <model>`: parse and print the program.
// `host_tests onnx <target> <model> <inputs file> <result file> [simplify_qdq]`: parse (and, when asked,
// run simplify_qdq as the mi355 target does on its own), evaluate with the parameter values of the
// inputs file (one line per parameter: name, then its values) and write every output value on a
// line of its own.  The Python tests drive it with the reference's ONNX test models.
static int onnx_tool(int argc, char** argv)
{
    if(argc != 4 and argc != 6 and argc != 7)
        return 2;
    auto p = migraphx::parse_onnx(argv[3]);
    if(argc == 7 and std::string(argv[6]) == "simplify_qdq")
        migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    if(std::string(argv[2]) == "print")
    {
        std::cout << p << std::endl;
        return 0;
    }
    if(argc < 6)
        return 2;
    std::ifstream in(argv[4]);
    migraphx::parameter_map params;
    std::string line;
    while(std::getline(in, line))
    {
        std::stringstream ls(line);
        std::string name;
        if(not(ls >> name))
            continue;
        std::vector<double> values;
        double v = 0;
        while(ls >> v)
            values.push_back(v);
        const auto s = p.get_parameter_shape(name);
        params[name] = argument{shape{s.type(), s.lens()}, values};
    }
    auto r = run_on(argv[2], p, params);
    std::ofstream out(argv[5]);
    out.precision(17);
    for(const auto& a : r)
        for(auto v : a.to_vector<double>())
            out << v << "\n";
    return 0;
}

int main(int argc, char** argv)
{
    try
    {
        if(argc > 1 and std::string(argv[1]) == "matmulnbits")
            return matmulnbits_tool(argc, argv);
        if(argc > 1 and std::string(argv[1]) == "onnx")
            return onnx_tool(argc, argv);
        return test::run(argc, argv);
    }
    catch(const std::exception& e)
    {
        std::cout << "error: " << e.what() << std::endl;
        return 4;
    }
}
