// GPU tests of the mi355 target: every program is compiled for the CPU oracle target and for
// "mi355" from the same host inputs, as the reference's test/verify/run_verify.cpp:139-226 does
// with `ref` and `gpu`.  Integer results and float results whose arithmetic the kernels reproduce
// exactly (int8 quant_dot with the dequantize epilogue, the int4 chain, float dot) must be
// bit-identical; fp8 results use the tolerances stated at the test.
#include "common.hpp"
#include "encoder.hpp"
#include "oracle_target.hpp"
#include "test.hpp"
#include <migraphx/load_save.hpp>
#include <chrono>
#include <cstdlib>
#include <fstream>
#include <thread>

using namespace testutil;
using migraphx::shape;

static void expect_same(const program& p, const migraphx::parameter_map& params)
{
    auto want = run_on("oracle", p, params);
    auto got  = run_on("mi355", p, params);
    EXPECT(want.size() == got.size());
    for(std::size_t i = 0; i < want.size(); i++)
    {
        if(not same_bytes(got[i], want[i]))
        {
            auto a = got[i].to_vector<double>();
            auto b = want[i].to_vector<double>();
            std::cout << "output " << i << " (" << want[i].get_shape() << " vs " << got[i].get_shape() << ")";
            for(std::size_t j = 0, shown = 0; j < std::min(a.size(), b.size()) and shown < 5; j++)
            {
                if(a[j] != b[j])
                {
                    std::cout << " [" << j << "] got " << a[j] << " want " << b[j];
                    shown++;
                }
            }
            std::cout << std::endl;
        }
        EXPECT(same_bytes(got[i], want[i]));
    }
    // parameters and results copied inside eval give the same answer
    auto got2 = run_on("mi355", p, params, true);
    for(std::size_t i = 0; i < want.size(); i++)
        EXPECT(same_bytes(got2[i], want[i]));
}

// The fp8 / block-scaled matrix-core instructions accumulate in fp32 where the CPU target holds the
// exact sum: the device result must stay within 1e-3 of the output's RMS, no element off by more
// than 2^-8 of the largest output.
static void expect_close_rms(const program& p, const migraphx::parameter_map& params)
{
    auto want_all = run_on("oracle", p, params);
    auto got_all  = run_on("mi355", p, params);
    EXPECT(want_all.size() == got_all.size());
    for(std::size_t o = 0; o < want_all.size(); o++)
    {
        auto want = want_all[o].to_vector<double>();
        auto got  = got_all[o].to_vector<double>();
        EXPECT(want.size() == got.size());
        double num = 0, den = 0, peak = 0, worst = 0;
        for(std::size_t i = 0; i < want.size(); i++)
        {
            num += (got[i] - want[i]) * (got[i] - want[i]);
            den += want[i] * want[i];
            peak  = std::max(peak, std::fabs(want[i]));
            worst = std::max(worst, std::fabs(got[i] - want[i]));
        }
        EXPECT(std::sqrt(num / den) < 1e-3);
        EXPECT(worst <= peak / 256);
    }
}

// The int4 kernel dequantizes every weight exactly as the reference does but accumulates the
// dot product in fp32 (v_dot2_f32_f16 partial sums, then a wavefront reduction) where the reference
// accumulates in double: outputs may differ by the last half-precision bit.  Allowed: one fp16
// step of the expected value, or 1e-3 relative, or 2e-4 absolute where the sum cancels.
static void expect_close_half(const program& p, const migraphx::parameter_map& params)
{
    auto want_all = run_on("oracle", p, params);
    auto got_all  = run_on("mi355", p, params);
    EXPECT(want_all.size() == got_all.size() and not want_all.empty());
    for(std::size_t r = 0; r < want_all.size(); r++)
    {
    const auto& want = want_all[r];
    const auto& got  = got_all[r];
    // (a result may be a strided view: a column slice of stacked projections)
    EXPECT(got.get_shape().lens() == want.get_shape().lens() and got.get_shape().type() == shape::half_type and
           want.get_shape().type() == shape::half_type);
    auto a = got.to_vector<double>();
    auto b = want.to_vector<double>();
    std::size_t exact = 0;
    for(std::size_t i = 0; i < a.size(); i++)
    {
        int e = 0;
        std::frexp(b[i], &e);
        const double ulp = std::ldexp(1.0, std::max(e - 11, -24));
        const double tol = std::max({ulp, 1e-3 * std::fabs(b[i]), 2e-4});
        if(not(std::fabs(a[i] - b[i]) <= tol))
            std::cout << "[" << i << "] got " << a[i] << " want " << b[i] << std::endl;
        EXPECT(std::fabs(a[i] - b[i]) <= tol);
        exact += a[i] == b[i] ? 1 : 0;
    }
    // the large majority is bit-identical
    EXPECT(exact * 10 >= a.size() * 8);
    }
}

static bool has_op(const program& p, const std::string& name)
{
    return count_ops(*p.get_main_module(), name) > 0;
}

// benchmark config 1: X fp32 [M, K] -> quantizelinear (scale 1/32, zp 0) -> int8; W int8 literal
// with per-output-channel scales; dot of the two dequantized tensors
static program qdq_matmul(std::size_t m,
                          std::size_t k,
                          std::size_t n,
                          bool weight_nk,
                          int zp_x,
                          int zp_w,
                          shape::type_t model_type,
                          unsigned seed)
{
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{model_type, {m, k}});
    auto xin = x;
    if(model_type != shape::float_type)
        xin = mm->add_instruction(make_op("convert", {{"target_type", shape::float_type}}), x);
    auto sx  = mm->add_literal(1.0f / 32);
    auto zx  = mm->add_literal(static_cast<std::int8_t>(zp_x));
    auto q   = add_quantize_op(*mm, "quantizelinear", xin, sx, zx);
    auto dx  = add_quantize_op(*mm, "dequantizelinear", q, sx, zx);
    std::vector<std::size_t> wl = weight_nk ? std::vector<std::size_t>{n, k} : std::vector<std::size_t>{k, n};
    auto w  = mm->add_literal(literal{shape{shape::int8_type, wl}, uniform_ints<int>(k * n, -127, 127, seed)});
    auto sw = mm->add_literal(literal{shape{shape::float_type, {n}}, uniform_floats(n, 0.001f, 0.01f, seed + 1)});
    auto zw = mm->add_literal(literal{shape{shape::int8_type, {n}}, std::vector<int>(n, zp_w)});
    const std::size_t axis = weight_nk ? 0 : 1;
    auto swb = mm->add_instruction(make_op("broadcast", {{"axis", axis}, {"out_lens", wl}}), sw);
    auto zwb = mm->add_instruction(make_op("broadcast", {{"axis", axis}, {"out_lens", wl}}), zw);
    instruction_ref dw = mm->add_instruction(make_op("dequantizelinear"), w, swb, zwb);
    if(weight_nk)
        dw = mm->add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), dw);
    if(model_type != shape::float_type)
    {
        dx = mm->add_instruction(make_op("convert", {{"target_type", model_type}}), dx);
        dw = mm->add_instruction(make_op("convert", {{"target_type", model_type}}), dw);
    }
    mm->add_return({mm->add_instruction(make_op("dot"), dx, dw)});
    return p;
}

TEST_CASE(config1_qdq_matmul)
{
    const std::size_t m = 256, k = 1024, n = 1024;
    auto p = qdq_matmul(m, k, n, false, 0, 0, shape::float_type, 0);
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    EXPECT(has_op(p, "quant_dot") and not has_op(p, "dot"));
    argument x{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 0)};
    expect_same(p, {{"x", x}});
    // the target runs simplify_qdq itself: the fake-quantized graph compiles to the same program
    auto raw  = qdq_matmul(m, k, n, false, 0, 0, shape::float_type, 0);
    auto got  = run_on("mi355", raw, {{"x", x}});
    auto want = run_on("oracle", p, {{"x", x}});
    EXPECT(same_bytes(got[0], want[0]));
    // one fused kernel instruction, nothing left of the zero-point or scale arithmetic
    program c = raw;
    c.compile(migraphx::make_target("mi355"));
    EXPECT(count_ops(*c.get_main_module(), "mi355::quant_dot") == 1);
    EXPECT(count_ops(*c.get_main_module(), "mi355::quantizelinear") == 1);
    EXPECT(not has_op(c, "mul") and not has_op(c, "dequantizelinear") and not has_op(c, "quant_dot"));
}

TEST_CASE(qdq_matmul_transposed_weight)
{
    const std::size_t m = 96, k = 320, n = 208;
    auto p = qdq_matmul(m, k, n, true, 0, 0, shape::float_type, 3);
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    argument x{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 4)};
    expect_same(p, {{"x", x}});
}

TEST_CASE(qdq_matmul_zero_points)
{
    const std::size_t m = 64, k = 256, n = 128;
    for(auto zp : {std::pair<int, int>{3, 0}, {0, -5}, {3, -5}, {-128, 127}})
    {
        auto p = qdq_matmul(m, k, n, false, zp.first, zp.second, shape::float_type, 5);
        migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
        argument x{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.5f, 6)};
        expect_same(p, {{"x", x}});
        program c = p;
        c.compile(migraphx::make_target("mi355"));
        // the three extra GEMMs of the zero-point terms became column / row sums
        EXPECT(count_ops(*c.get_main_module(), "mi355::quant_dot") == 1);
        EXPECT(not has_op(c, "add") and not has_op(c, "sub"));
    }
}

TEST_CASE(qdq_linear_layer_bias)
{
    // MatMul + Add of a [N] bias, as a linear layer is exported: the add joins the GEMM's epilogue
    // (one launch, no separate add) and the result stays bit-identical to the CPU target.  The
    // second shape has a zero point on the activations, the third an N that is no multiple of 4
    // (the any-stride kernel), the fourth a bias of shape [1, N] added from the left.
    struct layer
    {
        std::size_t m, k, n;
        int zp_x;
        bool weight_nk, left;
    };
    for(auto c : {layer{256, 768, 768, 0, true, false}, layer{64, 256, 128, 3, false, false},
                  layer{33, 96, 50, 0, false, false}, layer{128, 512, 3072, 0, true, true}})
    {
        auto p   = qdq_matmul(c.m, c.k, c.n, c.weight_nk, c.zp_x, 0, shape::float_type, 11);
        auto* mm = p.get_main_module();
        auto ret = std::prev(mm->end());
        auto y   = ret->inputs().front();
        std::vector<std::size_t> bl = c.left ? std::vector<std::size_t>{1, c.n} : std::vector<std::size_t>{c.n};
        auto b   = mm->add_literal(literal{shape{shape::float_type, bl}, normal_floats(c.n, 2.0f, 12)});
        auto bb  = mm->insert_instruction(ret, make_op("multibroadcast", {{"out_lens", {c.m, c.n}}}), b);
        auto sum = c.left ? mm->insert_instruction(ret, make_op("add"), bb, y)
                          : mm->insert_instruction(ret, make_op("add"), y, bb);
        migraphx::instruction::replace_argument(ret, y, sum);
        migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
        argument x{shape{shape::float_type, {c.m, c.k}}, normal_floats(c.m * c.k, 1.0f, 13)};
        expect_same(p, {{"x", x}});
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::quant_dot") == 1);
        EXPECT(not has_op(compiled, "mi355::binary") and not has_op(compiled, "mi355::chain"));
    }
    // a bias along the rows is no epilogue bias: it stays an add
    {
        const std::size_t m = 64, k = 128, n = 64;
        auto p   = qdq_matmul(m, k, n, false, 0, 0, shape::float_type, 14);
        auto* mm = p.get_main_module();
        auto ret = std::prev(mm->end());
        auto y   = ret->inputs().front();
        auto b   = mm->add_literal(literal{shape{shape::float_type, {m}}, normal_floats(m, 2.0f, 15)});
        auto bb  = mm->insert_instruction(ret, make_op("broadcast", {{"axis", 0}, {"out_lens", {m, n}}}), b);
        migraphx::instruction::replace_argument(ret, y, mm->insert_instruction(ret, make_op("add"), y, bb));
        migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
        argument x{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 16)};
        expect_same(p, {{"x", x}});
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        EXPECT(has_op(compiled, "mi355::binary"));
    }
}

TEST_CASE(qdq_linear_layers_share_activations)
{
    // Three linear layers of one shape over the same quantized activations (the q / k / v projections
    // of an attention block) and a fourth of another width: the three become one batched launch --
    // activations with a batch stride of 0, weights, column scales and biases stacked when the
    // program is compiled -- and each result is a dense block of the stacked one.  Bit-identical to
    // the CPU target, which evaluates the layers one by one.
    for(bool with_bias : {true, false})
    {
        const std::size_t m = 384, k = 256, n = 256;
        program p;
        auto* mm = p.get_main_module();
        auto x   = mm->add_parameter("x", shape{shape::float_type, {m, k}});
        auto sx  = mm->add_literal(1.0f / 32);
        auto zx  = mm->add_literal(static_cast<std::int8_t>(0));
        auto q   = add_quantize_op(*mm, "quantizelinear", x, sx, zx);
        auto dx  = add_quantize_op(*mm, "dequantizelinear", q, sx, zx);
        std::vector<instruction_ref> results;
        unsigned seed = 70;
        for(std::size_t width : {n, n, n, std::size_t{512}})
        {
            auto w  = mm->add_literal(literal{shape{shape::int8_type, {k, width}}, uniform_ints<int>(k * width, -127, 127, seed++)});
            auto sw = mm->add_literal(literal{shape{shape::float_type, {width}}, uniform_floats(width, 0.001f, 0.01f, seed++)});
            auto zw  = mm->add_literal(literal{shape{shape::int8_type, {width}}, std::vector<int>(width, 0)});
            auto swb = mm->add_instruction(make_op("broadcast", {{"axis", 1}, {"out_lens", {k, width}}}), sw);
            auto zwb = mm->add_instruction(make_op("broadcast", {{"axis", 1}, {"out_lens", {k, width}}}), zw);
            auto dw  = mm->add_instruction(make_op("dequantizelinear"), w, swb, zwb);
            instruction_ref y = mm->add_instruction(make_op("dot"), dx, dw);
            if(with_bias)
            {
                auto b  = mm->add_literal(literal{shape{shape::float_type, {width}}, normal_floats(width, 2.0f, seed++)});
                auto bb = mm->add_instruction(make_op("multibroadcast", {{"out_lens", {m, width}}}), b);
                y       = mm->add_instruction(make_op("add"), y, bb);
            }
            results.push_back(y);
        }
        mm->add_return(results);
        migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
        argument xa{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 69)};
        expect_same(p, {{"x", xa}});
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        if(count_ops(*compiled.get_main_module(), "mi355::quant_dot") != 2)
            std::cout << compiled << std::endl;
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::quant_dot") == 2);
        EXPECT(not has_op(compiled, "mi355::binary") and not has_op(compiled, "mi355::chain"));
        setenv("MIGRAPHX_MI355_DISABLE_SHARED_QUANT_DOT", "1", 1);
        program separate = p;
        separate.compile(migraphx::make_target("mi355"));
        unsetenv("MIGRAPHX_MI355_DISABLE_SHARED_QUANT_DOT");
        EXPECT(count_ops(*separate.get_main_module(), "mi355::quant_dot") == 4);
    }
}

TEST_CASE(qdq_linear_layer_skinny)
{
    // A few rows against a large weight matrix (decoding, small batches).  Up to 16 rows against
    // constant weights: the weights are reordered when the program is compiled and the layer is
    // one launch of mi355::quant_dot_prepacked.  More rows (or shapes the reordered form does not
    // take): the lowering hands mi355::quant_dot a workspace so that K is split over the chip, the
    // second kernel applies the epilogue; a layer with a short K gets no workspace.  All
    // bit-identical to the CPU target.
    struct layer
    {
        std::size_t m, k, n;
        int zp_x, zp_w;
        bool weight_nk, skinny, reordered;
        shape::type_t type;
    };
    for(auto c : {layer{16, 4096, 1024, 0, 0, true, true, true, shape::float_type},
                  layer{1, 2048, 512, 0, 0, false, true, true, shape::float_type},
                  layer{5, 1600, 304, 3, -2, false, true, true, shape::half_type},
                  layer{16, 1608, 304, 0, 0, false, false, false, shape::float_type}, // K % 64 != 0: neither form
                  layer{40, 1600, 304, 3, -2, false, true, false, shape::float_type},
                  layer{128, 3072, 768, 0, 0, true, true, false, shape::half_type},
                  layer{2048, 256, 1024, 0, 0, true, false, false, shape::float_type}})
    {
        auto p = qdq_matmul(c.m, c.k, c.n, c.weight_nk, c.zp_x, c.zp_w, c.type, 31);
        migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        const auto& mod = *compiled.get_main_module();
        EXPECT(count_ops(mod, "mi355::quant_dot_prepacked") == (c.reordered ? 1 : 0));
        EXPECT(count_ops(mod, "mi355::quant_dot") == (c.reordered ? 0 : 1));
        EXPECT(count_ops(mod, "mi355::quant_dot_prepack") == 0); // ran when the program was compiled
        for(auto ins = mod.begin(); ins != mod.end(); ++ins)
        {
            if(ins->name() != "mi355::quant_dot")
                continue;
            EXPECT(ins->get_operator().to_value().at("workspace").to<bool>() == c.skinny);
        }
        argument x{shape{c.type, {c.m, c.k}}, normal_floats(c.m * c.k, 1.0f, 32)};
        expect_same(p, {{"x", x}});
        // and after a round trip through a file
        if(c.reordered)
        {
            const std::string file = "/tmp/mi355_skinny_layer.mxr";
            migraphx::save(compiled, file);
            auto loaded = migraphx::load(file);
            // (compiled without offload_copy: parameters and results live in device memory)
            auto t  = migraphx::make_target("mi355");
            auto r1 = compiled.eval({{"x", t.copy_to(x)}});
            compiled.finish();
            auto r2 = loaded.eval({{"x", t.copy_to(x)}});
            loaded.finish();
            EXPECT(same_bytes(t.copy_from(r1[0]), t.copy_from(r2[0])));
            std::remove(file.c_str());
        }
    }
    // the bare product: int32 from int8 for few rows against a constant B, a variable B, more rows
    for(std::size_t rows : {12, 24})
    {
        program p;
        auto* mm = p.get_main_module();
        auto a   = mm->add_parameter("a", shape{shape::int8_type, {rows, 2048}});
        auto b   = mm->add_literal(literal{shape{shape::int8_type, {2048, 640}}, uniform_ints<std::int8_t>(2048 * 640, -128, 127, 33)});
        auto bv  = mm->add_parameter("b", shape{shape::int8_type, {2048, 640}});
        mm->add_return({mm->add_instruction(make_op("quant_dot"), a, b), mm->add_instruction(make_op("quant_dot"), a, bv)});
        argument av{shape{shape::int8_type, {rows, 2048}}, uniform_ints<std::int8_t>(rows * 2048, -128, 127, 34)};
        argument bb{shape{shape::int8_type, {2048, 640}}, uniform_ints<std::int8_t>(2048 * 640, -128, 127, 35)};
        expect_same(p, {{"a", av}, {"b", bb}});
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::quant_dot_prepacked") == (rows <= 16 ? 1 : 0));
        for(auto ins = compiled.get_main_module()->begin(); ins != compiled.get_main_module()->end(); ++ins)
            if(ins->name() == "mi355::quant_dot")
                EXPECT(ins->get_operator().to_value().at("workspace").to<bool>());
    }
}

// QDQ-wrapped convolution as a quantized ONNX model holds it: X float -> Q/DQ (one scale), W int8
// literal -> DQ with one scale per output channel, convolution of the two dequantized tensors
static program qdq_conv(std::vector<std::size_t> xl,
                        std::vector<std::size_t> wl,
                        const migraphx::operation& conv,
                        bool per_channel,
                        int zp_x,
                        shape::type_t model_type,
                        unsigned seed)
{
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{model_type, xl});
    auto xin = x;
    if(model_type != shape::float_type)
        xin = mm->add_instruction(make_op("convert", {{"target_type", shape::float_type}}), x);
    auto sx = mm->add_literal(1.0f / 16);
    auto zx = mm->add_literal(static_cast<std::int8_t>(zp_x));
    auto q  = add_quantize_op(*mm, "quantizelinear", xin, sx, zx);
    auto dx = add_quantize_op(*mm, "dequantizelinear", q, sx, zx);
    const std::size_t o = wl[0];
    std::size_t wn      = 1;
    for(auto l : wl)
        wn *= l;
    auto w  = mm->add_literal(literal{shape{shape::int8_type, wl}, uniform_ints<int>(wn, -127, 127, seed)});
    auto zw = mm->add_literal(std::int8_t{0});
    instruction_ref dw;
    if(per_channel)
    {
        auto sw  = mm->add_literal(literal{shape{shape::float_type, {o}}, uniform_floats(o, 0.001f, 0.01f, seed + 1)});
        auto swb = mm->add_instruction(make_op("broadcast", {{"axis", 0}, {"out_lens", wl}}), sw);
        auto zwb = mm->add_instruction(make_op("multibroadcast", {{"out_lens", wl}}), zw);
        dw       = mm->add_instruction(make_op("dequantizelinear"), w, swb, zwb);
    }
    else
    {
        auto sw = mm->add_literal(0.004f);
        dw      = add_quantize_op(*mm, "dequantizelinear", w, sw, zw);
    }
    if(model_type != shape::float_type)
    {
        dx = mm->add_instruction(make_op("convert", {{"target_type", model_type}}), dx);
        dw = mm->add_instruction(make_op("convert", {{"target_type", model_type}}), dw);
    }
    mm->add_return({mm->add_instruction(conv, dx, dw)});
    return p;
}

TEST_CASE(quant_convolution_programs)
{
    auto conv = [](std::vector<int64_t> padding, std::vector<int64_t> stride, std::vector<int64_t> dilation,
                   int64_t group, const std::string& name = "convolution") {
        return make_op(name, {{"padding", padding}, {"stride", stride}, {"dilation", dilation}, {"group", group}});
    };
    // bare quant_convolution, the shapes of test/ref/quant_convolution.cpp and of
    // test/verify/test_quant_conv*.cpp, int8 parameters: bit-exact int32
    struct bare
    {
        std::vector<std::size_t> xl, wl;
        std::vector<int64_t> padding, stride;
    };
    // and volumes: the shapes of test/ref/convolution.cpp:991-1060 and test/verify/test_conv3d.cpp
    for(const auto& c : {bare{{2, 3, 4, 4}, {2, 3, 3, 3}, {0, 0}, {1, 1}}, bare{{2, 3, 4, 4}, {2, 3, 3, 3}, {1, 1}, {2, 2}},
                         bare{{4, 3, 32, 32}, {16, 3, 5, 5}, {2, 2}, {1, 1}},
                         bare{{2, 3, 4, 4, 1}, {2, 3, 3, 3, 1}, {0, 0, 0}, {1, 1, 1}},
                         bare{{4, 3, 5, 5, 5}, {4, 3, 3, 3, 3}, {1, 0, 2}, {1, 2, 1}}})
    {
        program p;
        auto* mm = p.get_main_module();
        shape sx{shape::int8_type, c.xl};
        shape sw{shape::int8_type, c.wl};
        auto x = mm->add_parameter("x", sx);
        auto w = mm->add_parameter("w", sw);
        mm->add_return({mm->add_instruction(
            conv(c.padding, c.stride, std::vector<int64_t>(c.stride.size(), 1), 1, "quant_convolution"), x, w)});
        expect_same(p, {{"x", argument{sx, uniform_ints<int>(sx.elements(), -128, 127, 31)}},
                        {"w", argument{sw, uniform_ints<int>(sw.elements(), -128, 127, 32)}}});
    }
    // fake-quantized convolutions through simplify_qdq: one fused launch, bit-identical floats
    struct layer
    {
        std::vector<std::size_t> xl, wl;
        std::vector<int64_t> padding, stride, dilation;
        int64_t group;
        bool per_channel;
        shape::type_t model;
    };
    for(const auto& c : {layer{{2, 16, 14, 14}, {32, 16, 3, 3}, {1, 1}, {1, 1}, {1, 1}, 1, true, shape::float_type},
                         layer{{1, 3, 33, 31}, {8, 3, 7, 7}, {3, 3}, {2, 2}, {1, 1}, 1, true, shape::float_type},
                         layer{{2, 8, 10, 10}, {12, 2, 3, 3}, {2, 1}, {1, 2}, {2, 1}, 4, false, shape::float_type},
                         layer{{2, 16, 9, 9}, {16, 16, 1, 1}, {0, 0}, {1, 1}, {1, 1}, 1, true, shape::half_type},
                         layer{{2, 6, 40}, {10, 6, 5}, {2}, {3}, {1}, 1, true, shape::float_type},
                         // three spatial axes: per-channel scales, groups, low / high padding
                         layer{{2, 8, 6, 7, 5}, {12, 8, 3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {1, 1, 1}, 1, true, shape::float_type},
                         layer{{1, 32, 5, 6, 6}, {8, 16, 2, 3, 2}, {0, 1, 0, 1, 0, 1}, {1, 2, 1}, {2, 1, 1}, 2, false,
                               shape::float_type},
                         // SAME_UPPER-style padding: none in front, one behind
                         layer{{1, 8, 8, 8}, {8, 8, 3, 3}, {0, 0, 1, 1}, {2, 2}, {1, 1}, 1, true, shape::float_type}})
    {
        auto p = qdq_conv(c.xl, c.wl, conv(c.padding, c.stride, c.dilation, c.group), c.per_channel, 0, c.model, 41);
        migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
        EXPECT(has_op(p, "quant_convolution") and not has_op(p, "convolution"));
        shape sx{c.model, c.xl};
        expect_same(p, {{"x", argument{sx, normal_floats(sx.elements(), 2.0f, 42)}}});
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::quant_convolution") == 1);
        EXPECT(not has_op(compiled, "mi355::dequantizelinear") and not has_op(compiled, "mi355::binary"));
    }
    // a zero point on the activations adds a second quant_convolution (of the broadcast zero point:
    // the border it sees is zero-padded like the data's) and an int32 add; they stay separate
    // operators in front of a dequantizelinear with a tensor zero point
    for(int zp : {3, -7})
    {
        auto p = qdq_conv({2, 4, 8, 8}, {6, 4, 3, 3}, conv({1, 1}, {2, 1}, {1, 1}, 1), true, zp, shape::float_type, 43);
        migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
        EXPECT(count_ops(*p.get_main_module(), "quant_convolution") == 2);
        shape sx{shape::float_type, {2, 4, 8, 8}};
        expect_same(p, {{"x", argument{sx, normal_floats(sx.elements(), 2.0f, 44)}}});
    }
}

TEST_CASE(qdq_matmul_fp16_model)
{
    const std::size_t m = 48, k = 192, n = 80;
    auto p = qdq_matmul(m, k, n, false, 0, 0, shape::half_type, 7);
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    EXPECT(p.get_output_shapes().front().type() == shape::half_type);
    argument x{shape{shape::half_type, {m, k}}, normal_floats(m * k, 1.0f, 8)};
    expect_same(p, {{"x", x}});
}

TEST_CASE(bare_quant_dot_views)
{
    // the shapes of test/verify/test_batch_quant_dot_{1..5}.cpp and test_quant_dot_3args_*:
    // batches, transposed A, transposed B, both
    for(int variant = 0; variant < 4; variant++)
    {
        const bool ta = (variant & 1) != 0;
        const bool tb = (variant & 2) != 0;
        const std::size_t b0 = 3, b1 = 2, m = 24, k = 40, n = 56;
        program p;
        auto* mm = p.get_main_module();
        shape sa{shape::int8_type, ta ? std::vector<std::size_t>{b0, b1, k, m} : std::vector<std::size_t>{b0, b1, m, k}};
        shape sb{shape::int8_type, tb ? std::vector<std::size_t>{b0, b1, n, k} : std::vector<std::size_t>{b0, b1, k, n}};
        instruction_ref a = mm->add_parameter("a", sa);
        instruction_ref b = mm->add_parameter("b", sb);
        if(ta)
            a = mm->add_instruction(make_op("transpose", {{"permutation", {0, 1, 3, 2}}}), a);
        if(tb)
            b = mm->add_instruction(make_op("transpose", {{"permutation", {0, 1, 3, 2}}}), b);
        mm->add_return({mm->add_instruction(make_op("quant_dot"), a, b)});
        argument aa{sa, uniform_ints<int>(sa.elements(), -128, 127, 10 + variant)};
        argument ba{sb, uniform_ints<int>(sb.elements(), -128, 127, 20 + variant)};
        expect_same(p, {{"a", aa}, {"b", ba}});
    }
    // uint8 operands (op/quant_dot.hpp:62-64)
    {
        const std::size_t m = 33, k = 70, n = 21;
        program p;
        auto* mm = p.get_main_module();
        shape sa{shape::uint8_type, {m, k}};
        shape sb{shape::uint8_type, {k, n}};
        auto a = mm->add_parameter("a", sa);
        auto b = mm->add_parameter("b", sb);
        mm->add_return({mm->add_instruction(make_op("quant_dot"), a, b)});
        argument aa{sa, uniform_ints<int>(sa.elements(), 0, 255, 30)};
        argument ba{sb, uniform_ints<int>(sb.elements(), 0, 255, 31)};
        expect_same(p, {{"a", aa}, {"b", ba}});
    }
}

TEST_CASE(quant_dot_four_inputs)
{
    // the reference's known answer (test/ref/dot_op.cpp:1836-1865) on the device
    {
        program p;
        auto* mm = p.get_main_module();
        shape sa{shape::float_type, {2, 3}};
        shape sb{shape::float_type, {3, 2}};
        auto a  = mm->add_parameter("a", sa);
        auto b  = mm->add_parameter("b", sb);
        auto s1 = mm->add_literal(literal{sa, std::vector<float>{0.5f, 1, 0.5f, 1, 0.5f, 1}});
        auto s2 = mm->add_literal(literal{sb, std::vector<float>{1, 0.5f, 1, 0.5f, 1, 0.5f}});
        mm->add_return({mm->add_instruction(make_op("quant_dot"), a, b, s1, s2)});
        argument aa{sa, std::vector<float>{1, 2, 3, 4, 5, 6}};
        argument ba{sb, std::vector<float>{1, 2, 3, 4, 5, 6}};
        auto got = run_on("mi355", p, {{"a", aa}, {"b", ba}});
        EXPECT(got[0].to_vector<float>() == std::vector<float>{14.0f, 9.0f, 41.5f, 27.0f});
        expect_same(p, {{"a", aa}, {"b", ba}});
    }
    // fp8 operands with one power-of-two scale per block of 32 along K (the MX arrangement, scales
    // already spread over the elements), batched; A's scales arrive as a dense tensor, B's as a
    // broadcast view of one row.  B is row-major [K, N]: the lowering copies it into the
    // K-contiguous layout the block-scaled kernel reads.  The codes span the whole e4m3 range, so
    // the fp32 accumulation of the instruction shows: the fp8 tolerance, not bit equality.
    {
        const std::size_t bt = 2, m = 48, k = 64, n = 40;
        program p;
        auto* mm = p.get_main_module();
        shape sa{shape::fp8e4m3fn_type, {bt, m, k}};
        shape sb{shape::fp8e4m3fn_type, {bt, k, n}};
        shape ssa{shape::float_type, {bt, m, k}};
        shape ssb{shape::float_type, {n}};
        auto a   = mm->add_parameter("a", sa);
        auto b   = mm->add_parameter("b", sb);
        auto s1  = mm->add_parameter("sa", ssa);
        auto s2  = mm->add_parameter("sb", ssb);
        auto s2b = mm->add_instruction(make_op("broadcast", {{"axis", 2}, {"out_lens", {bt, k, n}}}), s2);
        mm->add_return({mm->add_instruction(make_op("quant_dot"), a, b, s1, s2b)});
        auto codes = [](std::size_t cnt, unsigned seed) {
            auto v = uniform_ints<int>(cnt, 0, 0x7d, seed);
            auto sg = uniform_ints<int>(cnt, 0, 1, seed + 1);
            std::vector<uint8_t> out(cnt);
            for(std::size_t i = 0; i < cnt; i++)
                out[i] = static_cast<uint8_t>(v[i] | (sg[i] << 7));
            return out;
        };
        std::vector<float> sav(ssa.elements());
        auto e1 = uniform_ints<int>(bt * m * (k / 32), -6, 3, 77);
        for(std::size_t i = 0; i < sav.size(); i++)
            sav[i] = std::ldexp(1.0f, e1[i / 32]);
        std::vector<float> sbv(n);
        auto e2 = uniform_ints<int>(n, -5, 2, 78);
        for(std::size_t i = 0; i < n; i++)
            sbv[i] = std::ldexp(1.0f, e2[i]);
        argument aa{sa};
        argument ba{sb};
        const auto ca = codes(sa.elements(), 70);
        const auto cb = codes(sb.elements(), 72);
        std::memcpy(aa.data(), ca.data(), ca.size());
        std::memcpy(ba.data(), cb.data(), cb.size());
        expect_close_rms(p, {{"a", aa}, {"b", ba}, {"sa", argument{ssa, sav}}, {"sb", argument{ssb, sbv}}});
        // a scale that is no power of two: the same graph, now bit for bit (exact path on the device)
        sbv[3] = 0.75f;
        expect_same(p, {{"a", aa}, {"b", ba}, {"sa", argument{ssa, sav}}, {"sb", argument{ssb, sbv}}});
        program c = p;
        c.compile(migraphx::make_target("mi355"));
        EXPECT(count_ops(*c.get_main_module(), "mi355::quant_dot_mx") == 1);
        EXPECT(not has_op(c, "quant_dot") and not has_op(c, "mi355::dot"));
    }
}

TEST_CASE(mx_fp4_matmul)
{
    // MX fp4: packed e2m1 operands, one power-of-two scale per 32 elements along K, as a graph of
    // unpack_fp4 -> dequantizelinear -> dot (test/simplify_qdq_test.cpp:1776-1860).  The target's
    // simplify_qdq turns it into the four-input quant_dot, which runs on the block-scaled
    // matrix-core kernel with the operands still packed.  Every product float(a) * scale is exact,
    // so the CPU target's result is the exact sum rounded once; the instruction accumulates in
    // fp32 (the tolerance of the fp8 quant_dot: 1e-3 of the output's RMS here, no element off by
    // more than 2^-8 of the largest).  With scales close together every partial sum is exact and
    // the results are the same bits.
    const std::size_t bt = 2, m = 40, k = 96, n = 24;
    shape pa{shape::fp4x2_type, {bt, m, k / 2}};
    shape pb{shape::fp4x2_type, {bt, n, k / 2}};
    shape sa{shape::float_type, {bt, m, k}};
    shape sb{shape::float_type, {bt, n, k}};
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
        auto tb  = mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 1}}}), db);
        mm->add_return({mm->add_instruction(make_op("dot"), da, tb)});
    }
    argument aa{pa};
    argument ba{pb};
    const auto ca = uniform_ints<uint8_t>(pa.elements(), 0, 255, 41);
    const auto cb = uniform_ints<uint8_t>(pb.elements(), 0, 255, 42);
    std::memcpy(aa.data(), ca.data(), ca.size());
    std::memcpy(ba.data(), cb.data(), cb.size());
    auto block_scales = [](std::size_t rows, std::size_t kk, int spread, unsigned seed) {
        auto e = uniform_ints<int>(rows * (kk / 32), -spread, spread, seed);
        std::vector<float> v(rows * kk);
        for(std::size_t i = 0; i < v.size(); i++)
            v[i] = std::ldexp(1.0f, e[i / 32]);
        return v;
    };
    for(int spread : {1, 5})
    {
        migraphx::parameter_map params = {{"a", aa}, {"b", ba}, {"sa", argument{sa, block_scales(bt * m, k, spread, 43)}},
                                          {"sb", argument{sb, block_scales(bt * n, k, spread, 44)}}};
        if(spread == 1)
        {
            expect_same(p, params);
            continue;
        }
        expect_close_rms(p, params);
    }
    // scales that are no powers of two: found on the device, evaluated as the operator is written
    {
        auto v1 = uniform_floats(sa.elements(), 0.25f, 2.0f, 46);
        auto v2 = uniform_floats(sb.elements(), 0.25f, 2.0f, 47);
        expect_same(p, {{"a", aa}, {"b", ba}, {"sa", argument{sa, v1}}, {"sb", argument{sb, v2}}});
    }
    program c = p;
    c.compile(migraphx::make_target("mi355"));
    EXPECT(count_ops(*c.get_main_module(), "mi355::quant_dot_mx") == 1);
    EXPECT(not has_op(c, "mi355::unpack_fp4") and not has_op(c, "mi355::dot"));
    EXPECT(not has_op(c, "dequantizelinear") and not has_op(c, "mi355::dequantizelinear"));
    // block scales that the graph spreads itself (one value per block, unsqueeze -> multibroadcast
    // -> reshape): the kernel gets the compact tensors
    program q;
    {
        auto* mm = q.get_main_module();
        auto a   = mm->add_parameter("a", pa);
        auto b   = mm->add_parameter("b", pb);
        auto s1  = mm->add_parameter("sa", shape{shape::float_type, {bt, m, k / 32}});
        auto s2  = mm->add_parameter("sb", shape{shape::float_type, {bt, n, k / 32}});
        auto spread32 = [&](instruction_ref x, std::size_t rows) {
            auto u  = mm->add_instruction(make_op("unsqueeze", {{"axes", {3}}}), x);
            auto mb = mm->add_instruction(make_op("multibroadcast", {{"out_lens", {bt, rows, k / 32, std::size_t{32}}}}), u);
            return mm->add_instruction(make_op("reshape", {{"dims", {static_cast<int64_t>(bt), static_cast<int64_t>(rows), static_cast<int64_t>(k)}}}), mb);
        };
        auto ua = mm->add_instruction(make_op("unpack_fp4"), a);
        auto ub = mm->add_instruction(make_op("unpack_fp4"), b);
        auto da = mm->add_instruction(make_op("dequantizelinear"), ua, spread32(s1, m));
        auto db = mm->add_instruction(make_op("dequantizelinear"), ub, spread32(s2, n));
        auto tb = mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 1}}}), db);
        mm->add_return({mm->add_instruction(make_op("dot"), da, tb)});
    }
    {
        auto compact = [](std::size_t count, unsigned seed) {
            auto e = uniform_ints<int>(count, -1, 1, seed);
            std::vector<float> v(count);
            for(std::size_t i = 0; i < count; i++)
                v[i] = std::ldexp(1.0f, e[i]);
            return v;
        };
        shape c1{shape::float_type, {bt, m, k / 32}};
        shape c2{shape::float_type, {bt, n, k / 32}};
        expect_same(q, {{"a", aa}, {"b", ba}, {"sa", argument{c1, compact(c1.elements(), 48)}},
                        {"sb", argument{c2, compact(c2.elements(), 49)}}});
        program qc = q;
        qc.compile(migraphx::make_target("mi355"));
        for(auto ins = qc.get_main_module()->begin(); ins != qc.get_main_module()->end(); ++ins)
            if(ins->name() == "mi355::quant_dot_mx")
            {
                EXPECT(ins->get_operator().to_value().at("sa_compact").to<bool>());
                EXPECT(ins->get_operator().to_value().at("sb_compact").to<bool>());
            }
        EXPECT(count_ops(*qc.get_main_module(), "mi355::quant_dot_mx") == 1);
    }
    // pack_fp4 on the device: float -> fp4x2 -> fp8, against the CPU target
    program r;
    {
        auto* mm = r.get_main_module();
        auto x   = mm->add_parameter("x", shape{shape::float_type, {16, 64}});
        auto pk  = mm->add_instruction(make_op("pack_fp4"), x);
        mm->add_return({pk, mm->add_instruction(make_op("unpack_fp4"), pk)});
    }
    expect_same(r, {{"x", argument{shape{shape::float_type, {16, 64}}, uniform_floats(16 * 64, -7.0f, 7.0f, 45)}}});
}

static void fp8_quantized_matmul_of(shape::type_t fp8_type, float fp8_max)
{
    // benchmark config 3 in small: activations and weights quantized to fp8 e4m3fn with amax-based
    // per-tensor scales, fp32 accumulation, bf16 output.  The fp8 MFMA instructions add each
    // group of 128 products with about 20 bits below the group's largest term, so the result is
    // not bit-identical to the oracle's exact sum: the error must stay within 1e-3 of the
    // output's RMS, and no element may be off by more than 2^-8 of the largest output (two bf16
    // steps at that magnitude).
    const std::size_t m = 128, k = 512, n = 256;
    auto xv = normal_floats(m * k, 1.0f, 30);
    auto wv = normal_floats(k * n, 0.02f, 31);
    float ax = 0, aw = 0;
    for(float v : xv)
        ax = std::max(ax, std::fabs(v));
    for(float v : wv)
        aw = std::max(aw, std::fabs(v));
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {m, k}});
    auto w   = mm->add_literal(literal{shape{shape::float_type, {k, n}}, wv});
    auto sx  = mm->add_literal(ax / fp8_max);
    auto sw  = mm->add_literal(aw / fp8_max);
    auto z   = mm->add_literal(literal{shape{fp8_type}, std::vector<float>{0.0f}});
    auto qx  = add_quantize_op(*mm, "quantizelinear", x, sx, z);
    auto dx  = add_quantize_op(*mm, "dequantizelinear", qx, sx, z);
    auto qw  = add_quantize_op(*mm, "quantizelinear", w, sw, z);
    auto dw  = add_quantize_op(*mm, "dequantizelinear", qw, sw, z);
    auto d   = mm->add_instruction(make_op("dot"), dx, dw);
    mm->add_return({mm->add_instruction(make_op("convert", {{"target_type", shape::bf16_type}}), d)});
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    EXPECT(has_op(p, "quant_dot") and not has_op(p, "dot"));
    argument xa{shape{shape::float_type, {m, k}}, xv};
    auto want = run_on("oracle", p, {{"x", xa}});
    auto got  = run_on("mi355", p, {{"x", xa}});
    EXPECT(got[0].get_shape().type() == shape::bf16_type);
    auto a = got[0].to_vector<double>();
    auto b = want[0].to_vector<double>();
    double num = 0, den = 0, peak = 0, worst = 0;
    for(std::size_t i = 0; i < a.size(); i++)
    {
        num += (a[i] - b[i]) * (a[i] - b[i]);
        den += b[i] * b[i];
        peak  = std::max(peak, std::fabs(b[i]));
        worst = std::max(worst, std::fabs(a[i] - b[i]));
    }
    EXPECT(std::sqrt(num / den) < 1e-3);
    EXPECT(worst <= peak / 256);
    // the weight was quantized once, at compile time
    program c = p;
    c.compile(migraphx::make_target("mi355"));
    EXPECT(count_ops(*c.get_main_module(), "mi355::quantizelinear") == 1);
    EXPECT(count_ops(*c.get_main_module(), "mi355::quant_dot") == 1);
    EXPECT(not has_op(c, "mi355::convert"));
}

// the MatMulNBits graph with random data (benchmark config 4 layout: block 128, zero point 8)
static program
matmulnbits_program(std::size_t m, std::size_t k, std::size_t n, std::size_t blk, bool with_zp, shape::type_t ft, unsigned seed)
{
    const std::size_t nblk = (k + blk - 1) / blk;
    program p;
    auto* mm = p.get_main_module();
    auto a   = mm->add_parameter("a", shape{ft, {m, k}});
    auto b   = mm->add_literal(literal{shape{shape::uint8_type, {n, nblk, blk / 2}}, uniform_ints<int>(n * nblk * blk / 2, 0, 255, seed)});
    auto s   = mm->add_literal(literal{shape{ft, {n * nblk}}, uniform_floats(n * nblk, 0.005f, 0.02f, seed + 1)});
    auto zp  = mm->end();
    if(with_zp)
        zp = mm->add_literal(literal{shape{shape::uint8_type, {n * ((nblk + 1) / 2)}}, uniform_ints<int>(n * ((nblk + 1) / 2), 0, 255, seed + 2)});
    mm->add_return({migraphx::op::builder::matmulnbits(*mm, a, b, s, zp, n, k, blk)});
    return p;
}

TEST_CASE(fp8_quantized_matmul) { fp8_quantized_matmul_of(shape::fp8e4m3fn_type, 448.0f); }

// the same graph over fp8 e5m2 (op/quant_dot.hpp:62-66 takes every fp8 type): two mantissa bits,
// so the quantization error is larger, but it is the oracle's too; the comparison is the same
TEST_CASE(fp8e5m2_quantized_matmul) { fp8_quantized_matmul_of(shape::fp8e5m2_type, 57344.0f); }

TEST_CASE(fp8e5m2_operators)
{
    // quantizelinear / dequantizelinear / convert / bare quant_dot on e5m2 tensors, bit for bit
    // (the bare product is small integers and halves: exact in the fp32 accumulator)
    const std::size_t m = 32, k = 64, n = 16;
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {m, k}});
    auto b   = mm->add_parameter("b", shape{shape::fp8e5m2_type, {k, n}});
    auto s   = mm->add_literal(0.37f);
    auto z   = mm->add_literal(literal{shape{shape::fp8e5m2_type}, std::vector<float>{1.5f}});
    auto q   = add_quantize_op(*mm, "quantizelinear", x, s, z);
    // (another scale than the quantizelinear's: simplify_qdq drops a pair that shares both)
    auto s2  = mm->add_literal(0.25f);
    auto dq  = add_quantize_op(*mm, "dequantizelinear", q, s2, z);
    auto cv  = mm->add_instruction(make_op("convert", {{"target_type", shape::fp8e5m2_type}}), x);
    auto ch  = mm->add_instruction(make_op("convert", {{"target_type", shape::half_type}}), cv);
    auto one = mm->add_literal(1.0f);
    auto z0  = mm->add_literal(literal{shape{shape::fp8e5m2_type}, std::vector<float>{0.0f}});
    auto y   = mm->add_parameter("y", shape{shape::float_type, {m, k}});
    auto qi  = add_quantize_op(*mm, "quantizelinear", y, one, z0);
    auto qd  = mm->add_instruction(make_op("quant_dot"), qi, b);
    mm->add_return({q, dq, cv, ch, qd});
    auto xi = uniform_ints<int>(m * k, -12, 12, 5);
    std::vector<float> xv(m * k);
    for(std::size_t i = 0; i < xv.size(); i++)
        xv[i] = 0.5f * static_cast<float>(xi[i]);
    const auto yv = xv;
    xv[3] = 1e9f;
    xv[4] = -1e9f;
    xv[5] = 1.52587890625e-05f * 1.5f;
    auto bi = uniform_ints<int>(k * n, -8, 8, 6);
    argument ba{shape{shape::fp8e5m2_type, {k, n}}, std::vector<float>(bi.begin(), bi.end())};
    EXPECT(ba.to_vector<float>()[7] == static_cast<float>(migraphx::fp8e5m2(static_cast<float>(bi[7]))));
    expect_same(p, {{"x", argument{shape{shape::float_type, {m, k}}, xv}},
                    {"y", argument{shape{shape::float_type, {m, k}}, yv}},
                    {"b", ba}});
    program c = p;
    c.compile(migraphx::make_target("mi355"));
    EXPECT(count_ops(*c.get_main_module(), "mi355::quant_dot") == 1);
}

TEST_CASE(int4_weight_only_gemv)
{
    // M = 1: the streaming kernel; the graph collapses into one instruction
    for(auto kn : {std::pair<std::size_t, std::size_t>{4096, 512}, {2048, 1000}})
    {
        auto p = matmulnbits_program(1, kn.first, kn.second, 128, false, shape::half_type, 40);
        argument a{shape{shape::half_type, {1, kn.first}}, normal_floats(kn.first, 1.0f, 41)};
        expect_close_half(p, {{"a", a}});
        program c = p;
        c.compile(migraphx::make_target("mi355"));
        // constant weights of a shape the reordered form takes (N % 16 == 0, K % 512 == 0) are
        // reordered when the program is compiled; the program keeps the reordered copy only
        const bool reordered = kn.second % 16 == 0 and kn.first % 512 == 0;
        EXPECT(count_ops(*c.get_main_module(), reordered ? "mi355::w4a16_gemm_prepacked" : "mi355::w4a16_gemm") == 1);
        EXPECT(not has_op(c, "mi355::w4a16_prepack"));
        EXPECT(not has_op(c, "mi355::dequantizelinear") and not has_op(c, "mi355::unpack_int4") and
               not has_op(c, "mi355::dot"));
        if(reordered)
        {
            EXPECT(count_ops(*c.get_main_module(), "mi355::literal") == 1);
            auto t  = migraphx::make_target("mi355");
            auto r1 = c.eval({{"a", t.copy_to(a)}});
            c.finish();
            auto loaded = migraphx::load_buffer(migraphx::save_buffer(c));
            auto r2     = loaded.eval({{"a", t.copy_to(a)}});
            loaded.finish();
            EXPECT(same_bytes(t.copy_from(r1[0]), t.copy_from(r2[0])));
        }
    }
}

TEST_CASE(int4_projections_sharing_activations)
{
    // q / k / v: three MatMulNBits of the same activations with constant weights become one launch
    // over the stacked weights; every result is a slice of it with the bits of its own launch
    for(std::size_t m : {1, 5})
    {
        const std::size_t k = 1024, blk = 128, nblk = k / blk;
        const std::vector<std::size_t> ns = {256, 64, 96};
        auto weights = [&](module& mod, std::size_t n, unsigned seed) {
            auto b = mod.add_literal(literal{shape{shape::uint8_type, {n, nblk, blk / 2}}, uniform_ints<int>(n * nblk * blk / 2, 0, 255, seed)});
            auto s = mod.add_literal(literal{shape{shape::half_type, {n * nblk}}, uniform_floats(n * nblk, 0.005f, 0.02f, seed + 1)});
            return std::make_pair(b, s);
        };
        program all;
        {
            auto* mm = all.get_main_module();
            auto a   = mm->add_parameter("a", shape{shape::half_type, {m, k}});
            std::vector<migraphx::instruction_ref> outs;
            for(std::size_t i = 0; i < ns.size(); i++)
            {
                auto ws = weights(*mm, ns[i], 70 + 10 * static_cast<unsigned>(i));
                outs.push_back(migraphx::op::builder::matmulnbits(*mm, a, ws.first, ws.second, mm->end(), ns[i], k, blk));
            }
            mm->add_return(outs);
        }
        argument a{shape{shape::half_type, {m, k}}, normal_floats(m * k, 1.0f, 69)};
        program c = all;
        c.compile(migraphx::make_target("mi355"));
        // (one row or a few rows of activations: the stacked constant weights are reordered at
        // compile time)
        EXPECT(count_ops(*c.get_main_module(), "mi355::w4a16_gemm_prepacked") == 1);
        EXPECT(count_ops(*c.get_main_module(), "mi355::w4a16_gemm") == 0);
        auto got = run_on("mi355", all, {{"a", a}});
        EXPECT(got.size() == ns.size());
        for(std::size_t i = 0; i < ns.size(); i++)
        {
            program one;
            auto* mm = one.get_main_module();
            auto ap  = mm->add_parameter("a", shape{shape::half_type, {m, k}});
            auto ws  = weights(*mm, ns[i], 70 + 10 * static_cast<unsigned>(i));
            mm->add_return({migraphx::op::builder::matmulnbits(*mm, ap, ws.first, ws.second, mm->end(), ns[i], k, blk)});
            expect_close_half(one, {{"a", a}});
            auto alone = run_on("mi355", one, {{"a", a}});
            EXPECT(alone.size() == 1 and got[i].get_shape().lens() == alone[0].get_shape().lens());
            EXPECT(got[i].to_vector<double>() == alone[0].to_vector<double>());
        }
    }
}

TEST_CASE(int4_projections_with_odd_column_counts_are_not_stacked)
{
    // A member's result becomes a column slice of the stacked product, and a kernel that takes such a
    // view as its activations reads 16 bytes at a time: projections whose column count is not a
    // multiple of 8 stay launches of their own and the others are stacked, wherever the odd one
    // stands.
    const std::size_t m = 5, k = 1024, blk = 128, nblk = k / blk;
    for(auto ns : {std::vector<std::size_t>{100, 64, 96}, std::vector<std::size_t>{64, 100, 96}})
    {
        program p;
        auto* mm = p.get_main_module();
        auto a   = mm->add_parameter("a", shape{shape::half_type, {m, k}});
        std::vector<migraphx::instruction_ref> outs;
        for(std::size_t i = 0; i < ns.size(); i++)
        {
            const auto n = ns[i];
            auto b = mm->add_literal(literal{shape{shape::uint8_type, {n, nblk, blk / 2}}, uniform_ints<int>(n * nblk * blk / 2, 0, 255, 170 + 10 * static_cast<unsigned>(i))});
            auto s = mm->add_literal(literal{shape{shape::half_type, {n * nblk}}, uniform_floats(n * nblk, 0.005f, 0.02f, 171 + 10 * static_cast<unsigned>(i))});
            outs.push_back(migraphx::op::builder::matmulnbits(*mm, a, b, s, mm->end(), n, k, blk));
        }
        mm->add_return(outs);
        program c = p;
        c.compile(migraphx::make_target("mi355"));
        // (the stacked pair has 160 columns and takes the reordered form, the odd one cannot)
        EXPECT(count_ops(*c.get_main_module(), "mi355::w4a16_gemm") == 1);
        EXPECT(count_ops(*c.get_main_module(), "mi355::w4a16_gemm_prepacked") == 1);
        argument av{shape{shape::half_type, {m, k}}, normal_floats(m * k, 1.0f, 169)};
        expect_close_half(p, {{"a", av}});
    }
}

TEST_CASE(int4_weight_only_gemm_small_batch)
{
    // constant weights, block size 128, a few rows that fit the LDS: the reordered form (as for one
    // row); K = 8192 takes 8 rows of it, 16 rows stay on mi355::w4a16_gemm
    for(auto mk : {std::pair<std::size_t, std::size_t>{2, 1024}, {16, 1024}, {8, 8192}, {16, 8192}})
    {
        const std::size_t m = mk.first, k = mk.second;
        auto p = matmulnbits_program(m, k, 384, 128, false, shape::half_type, 50);
        argument a{shape{shape::half_type, {m, k}}, normal_floats(m * k, 1.0f, 51)};
        expect_close_half(p, {{"a", a}});
        program c = p;
        c.compile(migraphx::make_target("mi355"));
        const bool reordered = not(m == 16 and k == 8192);
        EXPECT(count_ops(*c.get_main_module(), reordered ? "mi355::w4a16_gemm_prepacked" : "mi355::w4a16_gemm") == 1);
        EXPECT(not has_op(c, "mi355::w4a16_prepack"));
    }
    // per-block zero points packed two to a byte, block size 32
    auto p = matmulnbits_program(4, 512, 96, 32, true, shape::half_type, 52);
    argument a{shape{shape::half_type, {4, 512}}, normal_floats(4 * 512, 1.0f, 53)};
    expect_close_half(p, {{"a", a}});
    program c = p;
    c.compile(migraphx::make_target("mi355"));
    EXPECT(count_ops(*c.get_main_module(), "mi355::w4a16_gemm") == 1);
}

TEST_CASE(int4_weight_only_gemm_larger_batch)
{
    // more than 32 rows and N a multiple of 128: the tile kernel; where its column tiles do not
    // fill the chip the lowering adds a workspace and K is split (with packed zero points too)
    for(bool with_zp : {false, true})
    {
        auto p = matmulnbits_program(96, 2048, 256, 128, with_zp, shape::half_type, 54);
        argument a{shape{shape::half_type, {96, 2048}}, normal_floats(96 * 2048, 1.0f, 55)};
        expect_close_half(p, {{"a", a}});
        program c = p;
        c.compile(migraphx::make_target("mi355"));
        const auto& mod = *c.get_main_module();
        EXPECT(count_ops(mod, "mi355::w4a16_gemm") == 1);
        for(auto ins = mod.begin(); ins != mod.end(); ++ins)
            if(ins->name() == "mi355::w4a16_gemm")
                EXPECT(ins->get_operator().to_value().at("workspace").to<bool>());
    }
}

TEST_CASE(int4_weight_packed_along_axis_0_is_not_fused)
{
    // dot(a, transpose(dequantizelinear(unpack_int4{axis = 0}(w [N/2, K]), blockwise scales, 8))): the
    // same byte count as a weight packed along K, but the nibble pairs run along N.  The fused
    // kernel reads pairs along K, so this graph must go operator by operator, and match.
    const std::size_t m = 4, k = 256, n = 64, blk = 128;
    program p;
    auto* mm = p.get_main_module();
    auto a   = mm->add_parameter("a", shape{shape::half_type, {m, k}});
    auto w   = mm->add_literal(literal{shape{shape::uint8_type, {n / 2, k}}, uniform_ints<int>(n / 2 * k, 0, 255, 70)});
    auto s   = mm->add_literal(literal{shape{shape::half_type, {n, k / blk}}, uniform_floats(n * k / blk, 0.005f, 0.02f, 71)});
    auto u   = mm->add_instruction(migraphx::make_op("unpack_int4", {{"axis", 0}}), w);
    auto su  = mm->add_instruction(migraphx::make_op("unsqueeze", {{"axes", {2}}}), s);
    auto sb  = mm->add_instruction(migraphx::make_op("multibroadcast", {{"out_lens", {n, k / blk, blk}}}), su);
    auto sr  = mm->add_instruction(migraphx::make_op("reshape", {{"dims", {static_cast<int64_t>(n), -1}}}), sb);
    auto z   = mm->add_literal(literal{shape{shape::uint8_type, {1}}, std::vector<int>{8}});
    auto zb  = mm->add_instruction(migraphx::make_op("multibroadcast", {{"out_lens", {n, k}}}), z);
    auto dq  = mm->add_instruction(migraphx::make_op("dequantizelinear"), u, sr, zb);
    auto bt  = mm->add_instruction(migraphx::make_op("transpose", {{"permutation", {1, 0}}}), dq);
    mm->add_return({mm->add_instruction(migraphx::make_op("dot"), a, bt)});
    argument av{shape{shape::half_type, {m, k}}, normal_floats(m * k, 1.0f, 72)};
    expect_same(p, {{"a", av}});
    program c = p;
    c.compile(migraphx::make_target("mi355"));
    EXPECT(count_ops(*c.get_main_module(), "mi355::w4a16_gemm") == 0);
}

TEST_CASE(int4_unpack_pack_any_axis_programs)
{
    // unpack_int4 / pack_int4 along axis 0 and of a transposed view, as operators of a program
    for(int64_t axis : {0, 1})
    {
        program p;
        auto* mm = p.get_main_module();
        auto x   = mm->add_parameter("x", shape{shape::uint8_type, {6, 10}});
        auto xt  = mm->add_instruction(migraphx::make_op("transpose", {{"permutation", {1, 0}}}), x);
        auto u   = mm->add_instruction(migraphx::make_op("unpack_int4", {{"axis", axis}}), xt);
        auto pk  = mm->add_instruction(migraphx::make_op("pack_int4", {{"axis", 1 - axis}}), u);
        mm->add_return({u, pk});
        argument xv{shape{shape::uint8_type, {6, 10}}, uniform_ints<int>(60, 0, 255, 73)};
        expect_same(p, {{"x", xv}});
    }
}

TEST_CASE(int4_general_path)
{
    // float activations, or K that is not a multiple of the block: no fused kernel, the chain
    // runs operator by operator (the weight side once, at compile time) and still matches
    auto p = matmulnbits_program(5, 200, 48, 64, true, shape::float_type, 60);
    argument a{shape{shape::float_type, {5, 200}}, normal_floats(5 * 200, 1.0f, 61)};
    expect_same(p, {{"a", a}});
    program c = p;
    c.compile(migraphx::make_target("mi355"));
    EXPECT(count_ops(*c.get_main_module(), "mi355::dot") == 1);
    EXPECT(not has_op(c, "mi355::dequantizelinear")); // folded into a literal
}

TEST_CASE(quantize_int4_program)
{
    const std::size_t m = 8, k = 64, n = 96;
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {m, k}});
    auto w   = mm->add_literal(literal{shape{shape::float_type, {k, n}}, uniform_floats(k * n, -0.5f, 1.0f, 70)});
    mm->add_return({mm->add_instruction(make_op("dot"), x, w)});
    migraphx::quantize_int4_weights(p);
    argument xa{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 71)};
    expect_same(p, {{"x", xa}});
}

TEST_CASE(int8_calibration_on_device)
{
    const std::size_t m = 32, k = 128, n = 64;
    program fp;
    auto* mm = fp.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {m, k}});
    auto w   = mm->add_literal(literal{shape{shape::float_type, {k, n}}, normal_floats(k * n, 0.05f, 80)});
    mm->add_return({mm->add_instruction(make_op("dot"), x, w)});
    argument xa{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 81)};
    program on_oracle = fp;
    program on_device = fp;
    migraphx::quantize_int8(on_oracle, migraphx::make_target("oracle"), {{{"x", xa}}});
    migraphx::quantize_int8(on_device, migraphx::make_target("mi355"), {{{"x", xa}}});
    // same captured ranges, hence the same quantized program
    EXPECT(on_oracle == on_device);
    migraphx::run_passes(on_device, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    EXPECT(has_op(on_device, "quant_dot"));
    expect_same(on_device, {{"x", xa}});
    // and the float program itself runs on the device, bit-exact with the oracle's dot
    expect_same(fp, {{"x", xa}});
}

TEST_CASE(standalone_operators)
{
    // operators of the path outside any fused pattern
    const std::size_t r = 37, c = 50;
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {r, c}});
    auto s   = mm->add_literal(literal{shape{shape::float_type, {c}}, uniform_floats(c, 0.01f, 0.1f, 90)});
    auto z   = mm->add_literal(literal{shape{shape::int8_type, {c}}, uniform_ints<int>(c, -10, 10, 91)});
    std::vector<std::size_t> lens = {r, c};
    auto sb  = mm->add_instruction(make_op("broadcast", {{"axis", 1}, {"out_lens", lens}}), s);
    auto zb  = mm->add_instruction(make_op("broadcast", {{"axis", 1}, {"out_lens", lens}}), z);
    auto q   = mm->add_instruction(make_op("quantizelinear"), x, sb, zb);
    // a scale of its own, so that simplify_qdq does not cancel the pair
    auto s2  = mm->add_literal(literal{shape{shape::float_type, {c}}, uniform_floats(c, 0.01f, 0.1f, 93)});
    auto s2b = mm->add_instruction(make_op("broadcast", {{"axis", 1}, {"out_lens", lens}}), s2);
    auto dq  = mm->add_instruction(make_op("dequantizelinear"), q, s2b, zb);
    auto h   = mm->add_instruction(make_op("convert", {{"target_type", shape::half_type}}), dq);
    auto t   = mm->add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), q);
    auto ct  = mm->add_instruction(make_op("contiguous"), t);
    auto pk  = mm->add_instruction(make_op("pack_int4"), q);
    auto un  = mm->add_instruction(make_op("unpack_int4"), pk);
    mm->add_return({q, h, ct, pk, un});
    argument xa{shape{shape::float_type, {r, c}}, normal_floats(r * c, 1.0f, 92)};
    expect_same(p, {{"x", xa}});
}

TEST_CASE(concurrent_programs)
{
    // the reference's verify harness compiles and evaluates programs for several targets from
    // separate threads (test/verify/run_verify.cpp:46-58): registries are read-only after load, each
    // compiled program owns its context and stream
    const std::size_t m = 64, k = 256, n = 128;
    auto p = qdq_matmul(m, k, n, false, 2, -3, shape::float_type, 9);
    argument x{shape{shape::float_type, {m, k}}, normal_floats(m * k, 1.0f, 10)};
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    auto want = run_on("oracle", p, {{"x", x}});
    std::vector<int> ok(4, 0);
    std::vector<std::thread> threads;
    for(int t = 0; t < 4; t++)
        threads.emplace_back([&, t] {
            try
            {
                for(int rep = 0; rep < 3; rep++)
                {
                    auto got = run_on(t % 2 == 0 ? "mi355" : "oracle", p, {{"x", x}}, rep % 2 == 1 and t % 2 == 0);
                    if(not same_bytes(got[0], want[0]))
                        return;
                }
                ok[t] = 1;
            }
            catch(const std::exception& e)
            {
                std::cout << "thread " << t << ": " << e.what() << std::endl;
            }
        });
    for(auto& th : threads)
        th.join();
    for(int t = 0; t < 4; t++)
        EXPECT(ok[t] == 1);
}

TEST_CASE(no_host_fallback)
{
    // an operator without a kernel stops compilation instead of running on the host
    program p;
    auto* mm = p.get_main_module();
    auto x   = mm->add_parameter("x", shape{shape::float_type, {4, 4}});
    mm->add_return({mm->add_instruction(make_op("softmax", {{"axis", 0}}), x)});
    bool thrown = false;
    try
    {
        p.compile(migraphx::make_target("mi355"));
    }
    catch(const migraphx::exception& e)
    {
        thrown = std::string(e.what()).find("has no kernel") != std::string::npos;
    }
    EXPECT(thrown);
    // wrong parameter shape at eval
    program q;
    auto* qm = q.get_main_module();
    auto a   = qm->add_parameter("a", shape{shape::int8_type, {16, 64}});
    auto b   = qm->add_parameter("b", shape{shape::int8_type, {64, 16}});
    qm->add_return({qm->add_instruction(make_op("quant_dot"), a, b)});
    auto t = migraphx::make_target("mi355");
    q.compile(t);
    EXPECT(test::throws([&] { q.eval({{"a", t.allocate(shape{shape::int8_type, {16, 64}})}}); }));
    EXPECT(test::throws([&] {
        q.eval({{"a", t.allocate(shape{shape::int8_type, {16, 32}})},
                {"b", t.allocate(shape{shape::int8_type, {64, 16}})}});
    }));
}

TEST_CASE(float_dot_layouts)
{
    // op::dot on fp32 (bit-identical to gemm_naive's double accumulation): row-major and transposed
    // operands, sizes with ragged edges in every dimension, K not a multiple of 4, batches -- the
    // vector-load kernel, its element-wise edges and the generic kernel (odd leading dimension)
    struct dims { std::size_t b, m, n, k; };
    for(auto d : {dims{1, 64, 64, 16}, dims{3, 70, 66, 50}, dims{2, 130, 36, 19}, dims{1, 5, 7, 3}, dims{2, 96, 128, 64}})
    {
        for(int variant = 0; variant < 4; variant++)
        {
            const bool ta = (variant & 1) != 0;
            const bool tb = (variant & 2) != 0;
            program p;
            auto* mm = p.get_main_module();
            shape sa{shape::float_type, ta ? std::vector<std::size_t>{d.b, d.k, d.m} : std::vector<std::size_t>{d.b, d.m, d.k}};
            shape sb{shape::float_type, tb ? std::vector<std::size_t>{d.b, d.n, d.k} : std::vector<std::size_t>{d.b, d.k, d.n}};
            instruction_ref a = mm->add_parameter("a", sa);
            instruction_ref b = mm->add_parameter("b", sb);
            if(ta)
                a = mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 1}}}), a);
            if(tb)
                b = mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 1}}}), b);
            mm->add_return({mm->add_instruction(make_op("dot"), a, b)});
            // wide dynamic range so that a different summation order would show
            auto wide = [](std::size_t cnt, unsigned seed) {
                auto v = normal_floats(cnt, 1.0f, seed);
                auto e = uniform_ints<int>(cnt, -12, 12, seed + 1);
                for(std::size_t i = 0; i < cnt; i++)
                    v[i] = std::ldexp(v[i], e[i]);
                return v;
            };
            expect_same(p, {{"a", argument{sa, wide(sa.elements(), 90 + variant)}},
                            {"b", argument{sb, wide(sb.elements(), 95 + variant)}}});
        }
    }
}

TEST_CASE(float_dot_two_batch_axes)
{
    // The head split of an attention layer: q, k and v are [batch, rows, heads, width] tensors seen
    // as [batch, heads, rows, width] (k also with its last two axes swapped).  The two batch axes do
    // not collapse into one stride; the dot takes a stride for each instead of copies of the views.
    // Bit-identical to the CPU target; ragged sizes and a width that is not a multiple of 16.
    struct dims { std::size_t b, h, r, w; };
    for(auto d : {dims{2, 3, 40, 16}, dims{3, 2, 70, 20}, dims{1, 4, 64, 64}})
    {
        program p;
        auto* mm = p.get_main_module();
        shape s{shape::float_type, {d.b, d.r, d.h, d.w}};
        auto q  = mm->add_parameter("q", s);
        auto k  = mm->add_parameter("k", s);
        auto v  = mm->add_parameter("v", s);
        auto qh = mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 1, 3}}}), q);
        auto kt = mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 3, 1}}}), k);
        auto vh = mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 1, 3}}}), v);
        auto scores = mm->add_instruction(make_op("dot"), qh, kt);   // [b, h, r, r]
        auto ctx    = mm->add_instruction(make_op("dot"), scores, vh); // [b, h, r, w]
        mm->add_return({scores, ctx});
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::dot") == 2);
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::contiguous") == 0);
        expect_same(p, {{"q", argument{s, normal_floats(s.elements(), 1.0f, 61)}},
                        {"k", argument{s, normal_floats(s.elements(), 1.0f, 62)}},
                        {"v", argument{s, normal_floats(s.elements(), 1.0f, 63)}}});
    }
    // the same graph as exporters write it: a copy behind each head split, the keys transposed after
    // theirs.  None of the copies is made: the dots read the views.
    {
        const dims d{2, 4, 64, 32};
        program p;
        auto* mm = p.get_main_module();
        shape s{shape::float_type, {d.b, d.r, d.h, d.w}};
        auto split = [&](const std::string& name) {
            auto x = mm->add_parameter(name, s);
            auto t = mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 1, 3}}}), x);
            return mm->add_instruction(make_op("contiguous"), t);
        };
        auto qh = split("q");
        auto kh = split("k");
        auto vh = split("v");
        auto kt = mm->add_instruction(make_op("transpose", {{"permutation", {0, 1, 3, 2}}}), kh);
        auto scores = mm->add_instruction(make_op("dot"), qh, kt);
        auto ctx    = mm->add_instruction(make_op("dot"), scores, vh);
        // and the heads merged again behind the context: the dot writes that layout itself
        auto merged = mm->add_instruction(make_op("contiguous"),
                                          mm->add_instruction(make_op("transpose", {{"permutation", {0, 2, 1, 3}}}), ctx));
        auto flat = mm->add_instruction(make_op("reshape", {{"dims", {static_cast<int64_t>(d.b * d.r), static_cast<int64_t>(d.h * d.w)}}}), merged);
        mm->add_return({scores, flat});
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::dot") == 2);
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::contiguous") == 0);
        expect_same(p, {{"q", argument{s, normal_floats(s.elements(), 1.0f, 64)}},
                        {"k", argument{s, normal_floats(s.elements(), 1.0f, 65)}},
                        {"v", argument{s, normal_floats(s.elements(), 1.0f, 66)}}});
    }
}

TEST_CASE(dot_scale_epilogue)
{
    // attention scores: dot(q, k^T) * 1/sqrt(d) -- the multiplication joins the dot's store and the
    // result stays the two operators' (float(sum) rounded, then one fp32 multiplication)
    const std::size_t b = 3, h = 2, s = 48, d = 32;
    for(bool left : {false, true})
    {
        program p;
        auto* mm = p.get_main_module();
        shape sq{shape::float_type, {b, h, s, d}};
        auto q   = mm->add_parameter("q", sq);
        auto k   = mm->add_parameter("k", sq);
        auto kt  = mm->add_instruction(make_op("transpose", {{"permutation", {0, 1, 3, 2}}}), k);
        auto qk  = mm->add_instruction(make_op("dot"), q, kt);
        auto c   = mm->add_literal(literal{shape{shape::float_type, {1}}, std::vector<float>{0.17677669f}});
        auto cb  = mm->add_instruction(make_op("multibroadcast", {{"out_lens", qk->get_shape().lens()}}), c);
        auto sc  = left ? mm->add_instruction(make_op("mul"), cb, qk) : mm->add_instruction(make_op("mul"), qk, cb);
        mm->add_return({mm->add_instruction(make_op("softmax", {{"axis", 3}}), sc)});
        migraphx::parameter_map params{{"q", argument{sq, normal_floats(sq.elements(), 1.0f, 61)}},
                                       {"k", argument{sq, normal_floats(sq.elements(), 1.0f, 62)}}};
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::dot") == 1);
        EXPECT(not has_op(compiled, "mi355::binary") and not has_op(compiled, "mi355::chain"));
        auto want = run_on("oracle", p, params);
        auto got  = run_on("mi355", p, params);
        EXPECT(max_rel_diff(got[0], want[0], 1e-30) < 4e-6);
        // the scaled scores themselves are bit-identical
        program scores;
        auto* sm = scores.get_main_module();
        auto q2  = sm->add_parameter("q", sq);
        auto k2  = sm->add_parameter("k", sq);
        auto kt2 = sm->add_instruction(make_op("transpose", {{"permutation", {0, 1, 3, 2}}}), k2);
        auto qk2 = sm->add_instruction(make_op("dot"), q2, kt2);
        auto c2  = sm->add_literal(literal{shape{shape::float_type, {1}}, std::vector<float>{0.17677669f}});
        auto cb2 = sm->add_instruction(make_op("multibroadcast", {{"out_lens", qk2->get_shape().lens()}}), c2);
        sm->add_return({left ? sm->add_instruction(make_op("mul"), cb2, qk2)
                             : sm->add_instruction(make_op("mul"), qk2, cb2)});
        expect_same(scores, params);
    }
    // a dot with a second user keeps its own result: nothing is fused
    {
        program p;
        auto* mm = p.get_main_module();
        shape sa{shape::float_type, {16, 24}};
        shape sb{shape::float_type, {24, 8}};
        auto a  = mm->add_parameter("a", sa);
        auto bb = mm->add_parameter("b", sb);
        auto ab = mm->add_instruction(make_op("dot"), a, bb);
        auto c  = mm->add_literal(literal{shape{shape::float_type, {1}}, std::vector<float>{3.0f}});
        auto cb = mm->add_instruction(make_op("multibroadcast", {{"out_lens", ab->get_shape().lens()}}), c);
        auto sc = mm->add_instruction(make_op("mul"), ab, cb);
        mm->add_return({mm->add_instruction(make_op("add"), sc, ab)});
        expect_same(p, {{"a", argument{sa, normal_floats(sa.elements(), 1.0f, 63)}},
                        {"b", argument{sb, normal_floats(sb.elements(), 1.0f, 64)}}});
    }
}

TEST_CASE(float_operators)
{
    // the float operators around the GEMMs, one by one against the CPU target: exact where the
    // arithmetic is IEEE (add / sub / mul / div / sqrt / rsqrt, gather), within a few units in the
    // last place where a math-library function or the summation order is involved
    const std::size_t r = 33, c = 200;
    auto run = [&](const std::function<instruction_ref(module&, instruction_ref, instruction_ref)>& f, bool exact) {
        static int case_no = 0;
        case_no++;
        program p;
        auto* mm = p.get_main_module();
        auto x   = mm->add_parameter("x", shape{shape::float_type, {r, c}});
        auto y   = mm->add_parameter("y", shape{shape::float_type, {r, c}});
        mm->add_return({f(*mm, x, y)});
        argument xa{shape{shape::float_type, {r, c}}, normal_floats(r * c, 2.0f, 100)};
        argument ya{shape{shape::float_type, {r, c}}, uniform_floats(r * c, 0.5f, 3.0f, 101)};
        auto want = run_on("oracle", p, {{"x", xa}, {"y", ya}});
        auto got  = run_on("mi355", p, {{"x", xa}, {"y", ya}});
        if(not(exact ? same_bytes(got[0], want[0]) : max_rel_diff(got[0], want[0], 1e-30) < 4e-6))
            std::cout << "float operator case " << case_no << ": max rel diff "
                      << max_rel_diff(got[0], want[0], 1e-30) << std::endl;
        if(exact)
            EXPECT(same_bytes(got[0], want[0]));
        else
            EXPECT(max_rel_diff(got[0], want[0], 1e-30) < 4e-6);
    };
    for(auto name : {"add", "sub", "mul", "div"})
        run([&](module& m, instruction_ref x, instruction_ref y) { return m.add_instruction(make_op(name), x, y); }, true);
    // broadcast operands: a row vector and a column of means
    run([&](module& m, instruction_ref x, instruction_ref) {
        auto mean = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), x);
        auto mb   = m.add_instruction(make_op("multibroadcast", {{"out_lens", x->get_shape().lens()}}), mean);
        return m.add_instruction(make_op("sub"), x, mb);
    }, false);
    run([&](module& m, instruction_ref, instruction_ref y) { return m.add_instruction(make_op("sqrt"), y); }, true);
    run([&](module& m, instruction_ref, instruction_ref y) { return m.add_instruction(make_op("rsqrt"), y); }, true);
    for(auto name : {"erf", "exp", "tanh"})
        run([&](module& m, instruction_ref x, instruction_ref) { return m.add_instruction(make_op(name), x); }, false);
    run([&](module& m, instruction_ref x, instruction_ref) { return m.add_instruction(make_op("softmax", {{"axis", 1}}), x); }, false);
    // gather rows, negative index included
    program p;
    auto* mm = p.get_main_module();
    auto t   = mm->add_literal(literal{shape{shape::float_type, {50, 24}}, normal_floats(50 * 24, 1.0f, 102)});
    auto i   = mm->add_parameter("i", shape{shape::int32_type, {7}});
    mm->add_return({mm->add_instruction(make_op("gather", {{"axis", 0}}), t, i)});
    argument ia{shape{shape::int32_type, {7}}, std::vector<int>{0, 49, 3, 3, -1, 17, -50}};
    expect_same(p, {{"i", ia}});
}

TEST_CASE(narrow_type_operators_and_float_convolution)
{
    // What the integer-MatMul / QLinearConv front ends leave in a graph besides the GEMMs: add / sub /
    // mul on int8, uint8 (wrapping) and half, bf16 (the operator on floats, the result truncated),
    // convert to the integer types (NaN -> 0, saturating, truncating), and a float convolution --
    // each bit for bit against the CPU target.
    const std::size_t r = 19, c = 77;
    for(auto t : {shape::int8_type, shape::uint8_type, shape::half_type, shape::bf16_type})
    {
        const bool integer = t == shape::int8_type or t == shape::uint8_type;
        for(auto name : {"add", "sub", "mul", "div"})
        {
            if(integer and std::string(name) == "div")
                continue;
            program p;
            auto* mm = p.get_main_module();
            auto x   = mm->add_parameter("x", shape{t, {r, c}});
            auto y   = mm->add_parameter("y", shape{t, {c}});
            auto yb  = mm->add_instruction(make_op("multibroadcast", {{"out_lens", {r, c}}}), y);
            auto z   = mm->add_literal(literal{shape{t}, std::vector<float>{3.0f}});
            auto zb  = mm->add_instruction(make_op("multibroadcast", {{"out_lens", {r, c}}}), z);
            auto v   = mm->add_instruction(make_op(name), x, yb);
            mm->add_return({mm->add_instruction(make_op(name), v, zb)});
            std::vector<float> xv, yv;
            if(integer)
            {
                const int lo = t == shape::int8_type ? -128 : 0, hi = t == shape::int8_type ? 127 : 255;
                auto xi = uniform_ints<int>(r * c, lo, hi, 400);
                auto yi = uniform_ints<int>(c, lo, hi, 401);
                xv.assign(xi.begin(), xi.end());
                yv.assign(yi.begin(), yi.end());
            }
            else
            {
                xv = normal_floats(r * c, 30.0f, 402);
                yv = uniform_floats(c, 0.01f, 5.0f, 403);
            }
            expect_same(p, {{"x", argument{shape{t, {r, c}}, xv}}, {"y", argument{shape{t, {c}}, yv}}});
        }
    }
    {
        program p;
        auto* mm = p.get_main_module();
        auto x   = mm->add_parameter("x", shape{shape::float_type, {r, c}});
        std::vector<instruction_ref> outs;
        for(auto t : {shape::int8_type, shape::uint8_type, shape::int32_type})
            outs.push_back(mm->add_instruction(make_op("convert", {{"target_type", t}}), x));
        auto h = mm->add_instruction(make_op("convert", {{"target_type", shape::half_type}}), x);
        outs.push_back(mm->add_instruction(make_op("convert", {{"target_type", shape::int8_type}}), h));
        mm->add_return(outs);
        auto xv = normal_floats(r * c, 90.0f, 404);
        xv[0]   = std::numeric_limits<float>::quiet_NaN();
        xv[1]   = std::numeric_limits<float>::infinity();
        xv[2]   = -std::numeric_limits<float>::infinity();
        xv[3]   = 3e9f;
        xv[4]   = -3e9f;
        xv[5]   = 127.9f;
        xv[6]   = -128.9f;
        xv[7]   = -0.9f;
        xv[8]   = 255.5f;
        expect_same(p, {{"x", argument{shape{shape::float_type, {r, c}}, xv}}});
    }
    // float convolution: groups, strides, dilation, padding on one side more than on the other, one
    // to three spatial axes
    struct conv_case
    {
        std::vector<std::size_t> x, w;
        std::vector<int64_t> pad, stride, dil;
        int64_t group;
    };
    for(auto k : {conv_case{{2, 6, 11, 9}, {8, 3, 3, 2}, {1, 0, 2, 1}, {2, 1}, {1, 2}, 2},
                  conv_case{{1, 3, 20}, {5, 3, 4}, {2}, {3}, {1}, 1},
                  conv_case{{1, 4, 5, 6, 7}, {4, 1, 2, 3, 3}, {0, 1, 1}, {1, 2, 1}, {2, 1, 1}, 4}})
    {
        program p;
        auto* mm = p.get_main_module();
        auto x   = mm->add_parameter("x", shape{shape::float_type, k.x});
        std::size_t wn = 1;
        for(auto l : k.w)
            wn *= l;
        auto w = mm->add_literal(literal{shape{shape::float_type, k.w}, normal_floats(wn, 0.5f, 405)});
        mm->add_return({mm->add_instruction(
            make_op("convolution", {{"padding", k.pad}, {"stride", k.stride}, {"dilation", k.dil}, {"group", k.group}}),
            x, w)});
        std::size_t xn = 1;
        for(auto l : k.x)
            xn *= l;
        expect_same(p, {{"x", argument{shape{shape::float_type, k.x}, normal_floats(xn, 1.0f, 406)}}});
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::convolution") == 1);
    }
}

TEST_CASE(intermediate_buffers_share_one_arena)
{
    // memory_coloring: the buffers of a compiled program are places in one block of device memory,
    // shared by buffers whose lives do not overlap.  A long chain of matrix products (each needs
    // the one before it only) must come out the size of a few buffers, not of all of them; an early
    // result that is returned must survive everything computed after it; a view of a buffer keeps
    // the buffer alive; and the results are those of the program with a buffer per instruction.
    const std::size_t n = 96;
    program p;
    auto* mm = p.get_main_module();
    shape s{shape::float_type, {n, n}};
    auto x     = mm->add_parameter("x", s);
    auto w     = mm->add_literal(literal{s, normal_floats(n * n, 0.1f, 901)});
    auto early = mm->add_instruction(make_op("dot"), x, w);
    auto early_t = mm->add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), early);
    auto y     = early;
    for(int i = 0; i < 12; i++)
        y = mm->add_instruction(make_op("dot"), y, w);
    auto late = mm->add_instruction(make_op("dot"), early_t, y); // the view of `early`, read at the end
    mm->add_return({early, y, late});
    argument xa{s, normal_floats(n * n, 1.0f, 902)};

    program colored = p;
    colored.compile(migraphx::make_target("mi355"));
    const auto& mod = *colored.get_main_module();
    EXPECT(count_ops(mod, "mi355::arena") == 1 and count_ops(mod, "mi355::allocate") == 0);
    EXPECT(count_ops(mod, "mi355::load") >= 14);
    std::size_t arena_bytes = 0;
    for(auto ins = mod.begin(); ins != mod.end(); ++ins)
        if(ins->name() == "mi355::arena")
            arena_bytes = ins->get_shape().bytes();
    // 14 products of 36 KiB: `early`, the two last results and one or two buffers in rotation
    EXPECT(arena_bytes >= 3 * n * n * 4 and arena_bytes <= 6 * n * n * 4);

    auto got = run_on("mi355", p, {{"x", xa}});
    setenv("MIGRAPHX_MI355_DISABLE_MEMORY_COLORING", "1", 1);
    program plain = p;
    plain.compile(migraphx::make_target("mi355"));
    auto want = run_on("mi355", p, {{"x", xa}});
    unsetenv("MIGRAPHX_MI355_DISABLE_MEMORY_COLORING");
    EXPECT(count_ops(*plain.get_main_module(), "mi355::arena") == 0 and
           count_ops(*plain.get_main_module(), "mi355::allocate") >= 14);
    EXPECT(got.size() == 3 and want.size() == 3);
    for(std::size_t i = 0; i < 3; i++)
        EXPECT(same_bytes(got[i], want[i]));
    auto cpu = run_on("oracle", p, {{"x", xa}});
    for(std::size_t i = 0; i < 3; i++)
        EXPECT(same_bytes(got[i], cpu[i]));
    // a saved and reloaded program keeps its places
    auto loaded = migraphx::load_buffer(migraphx::save_buffer(colored));
    auto t      = migraphx::make_target("mi355");
    auto again  = loaded.eval({{"x", t.copy_to(xa)}});
    loaded.finish();
    for(std::size_t i = 0; i < 3; i++)
        EXPECT(same_bytes(t.copy_from(again[i]), got[i]));
}

TEST_CASE(chain_quantized_for_the_next_layer)
{
    // A float chain whose only reader is a per-tensor quantizelinear to int8 (the activations in
    // front of a quantized layer) is one mi355::chain_q8; a chain that something else reads too
    // keeps its float result and the quantizelinear stays a kernel of its own.  Both equal the CPU
    // target byte for byte (IEEE-exact operators in the chain).
    for(bool second_reader : {false, true})
        for(bool with_zero_point : {false, true})
        {
            const std::size_t r = 70, c = 328;
            program p;
            auto* mm = p.get_main_module();
            shape s{shape::float_type, {r, c}};
            auto x  = mm->add_parameter("x", s);
            auto y  = mm->add_parameter("y", s);
            auto v  = mm->add_literal(literal{shape{shape::float_type, {c}}, uniform_floats(c, 0.5f, 2.0f, 77)});
            auto vb = mm->add_instruction(make_op("multibroadcast", {{"out_lens", s.lens()}}), v);
            auto t  = mm->add_instruction(make_op("mul"), mm->add_instruction(make_op("add"), x, y), vb);
            auto sc = mm->add_literal(literal{shape{shape::float_type}, std::vector<float>{0.0625f}});
            auto sb = mm->add_instruction(make_op("multibroadcast", {{"out_lens", s.lens()}}), sc);
            std::vector<instruction_ref> qargs{t, sb};
            if(with_zero_point)
            {
                auto z = mm->add_literal(literal{shape{shape::int8_type}, std::vector<float>{-5.0f}});
                qargs.push_back(mm->add_instruction(make_op("multibroadcast", {{"out_lens", s.lens()}}), z));
            }
            // without a zero point the operator's result type is its out_type attribute
            auto q = mm->add_instruction(make_op("quantizelinear", {{"out_type", shape::int8_type}}), qargs);
            if(second_reader)
                mm->add_return({q, mm->add_instruction(make_op("sub"), t, y)});
            else
                mm->add_return({q});
            program compiled = p;
            compiled.compile(migraphx::make_target("mi355"));
            const auto& mod = *compiled.get_main_module();
            EXPECT(count_ops(mod, "mi355::chain_q8") == (second_reader ? 0u : 1u));
            EXPECT(count_ops(mod, "mi355::quantizelinear") == (second_reader ? 1u : 0u));
            argument xa{s, normal_floats(r * c, 3.0f, 78)};
            argument ya{s, normal_floats(r * c, 3.0f, 79)};
            expect_same(p, {{"x", xa}, {"y", ya}});
        }
}

TEST_CASE(pointwise_chains)
{
    // Chains of float operators become one mi355::chain each.  With IEEE-exact operators the fused
    // program must equal the CPU target bit for bit; with erf in the chain it must equal the
    // unfused mi355 program bit for bit (same device functions, same order) and the CPU target
    // within the math library's few units in the last place.
    using builder = std::function<instruction_ref(module&, instruction_ref, instruction_ref, instruction_ref)>;
    struct counts
    {
        std::size_t chains, singles, row_chains = 0;
    };
    auto run = [&](std::size_t r, std::size_t c, const builder& f, bool exact, counts expected) {
        static int case_no = 0;
        case_no++;
        program p;
        auto* mm = p.get_main_module();
        shape s{shape::float_type, {r, c}};
        auto x = mm->add_parameter("x", s);
        auto y = mm->add_parameter("y", s);
        auto v = mm->add_parameter("v", shape{shape::float_type, {c}});
        mm->add_return({f(*mm, x, y, v)});
        migraphx::parameter_map params{{"x", argument{s, normal_floats(r * c, 2.0f, 300 + case_no)}},
                                       {"y", argument{s, uniform_floats(r * c, 0.5f, 3.0f, 400 + case_no)}},
                                       {"v", argument{shape{shape::float_type, {c}}, uniform_floats(c, 0.5f, 2.0f, 500 + case_no)}}};
        program compiled = p;
        compiled.compile(migraphx::make_target("mi355"));
        const auto chains  = count_ops(*compiled.get_main_module(), "mi355::chain");
        const auto singles = count_ops(*compiled.get_main_module(), "mi355::binary") +
                             count_ops(*compiled.get_main_module(), "mi355::unary");
        if(chains != expected.chains or singles != expected.singles)
            std::cout << "chain case " << case_no << ": " << chains << " chains, " << singles << " single operators"
                      << std::endl;
        EXPECT(chains == expected.chains);
        EXPECT(singles == expected.singles);
        EXPECT(count_ops(*compiled.get_main_module(), "mi355::chain_rows") == expected.row_chains);
        auto got = run_on("mi355", p, params);
        setenv("MIGRAPHX_DISABLE_POINTWISE_FUSION", "1", 1);
        program plain = p;
        plain.compile(migraphx::make_target("mi355"));
        auto unfused = run_on("mi355", p, params);
        unsetenv("MIGRAPHX_DISABLE_POINTWISE_FUSION");
        EXPECT(not has_op(plain, "mi355::chain"));
        EXPECT(not has_op(plain, "mi355::chain_rows"));
        EXPECT(same_bytes(got[0], unfused[0]));
        auto want = run_on("oracle", p, params);
        if(exact)
        {
            if(not same_bytes(got[0], want[0]))
                std::cout << "chain case " << case_no << " differs from the CPU target, max rel diff "
                          << max_rel_diff(got[0], want[0], 1e-30) << std::endl;
            EXPECT(same_bytes(got[0], want[0]));
        }
        else
        {
            // 1 + erf(x) cancels for negative x, so small results carry the math library's
            // absolute error: relative to max(|expected|, 0.25)
            if(not(max_rel_diff(got[0], want[0], 0.25) < 4e-6))
                std::cout << "chain case " << case_no << ": max rel diff " << max_rel_diff(got[0], want[0], 0.25)
                          << std::endl;
            EXPECT(max_rel_diff(got[0], want[0], 0.25) < 4e-6);
        }
    };
    auto op = [](module& m, const std::string& name, auto... args) { return m.add_instruction(make_op(name), args...); };
    auto bcast = [](module& m, instruction_ref v, instruction_ref like) {
        return m.add_instruction(make_op("multibroadcast", {{"out_lens", like->get_shape().lens()}}), v);
    };
    // bias + residual
    run(33, 200, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref v) {
        return op(m, "add", op(m, "add", x, bcast(m, v, x)), y);
    }, true, {1, 0});
    // the tail of layer normalisation: (x / sigma) * gamma + beta with a per-row sigma
    run(33, 200, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref v) {
        auto var   = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), op(m, "mul", y, y));
        auto sigma = bcast(m, op(m, "sqrt", var), x);
        return op(m, "add", op(m, "mul", op(m, "div", x, sigma), bcast(m, v, x)), bcast(m, v, x));
    }, false, {1, 2});
    // an operand used on both sides, and the reversed forms of sub and div
    run(16, 64, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref) {
        auto sq = op(m, "mul", x, x);
        return op(m, "div", y, op(m, "sub", y, op(m, "neg", sq)));
    }, true, {1, 0});
    // two computed operands: the first is saved while the second is evaluated
    run(16, 64, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref) {
        return op(m, "div", op(m, "add", x, y), op(m, "sqrt", op(m, "add", y, y)));
    }, true, {1, 0});
    run(16, 64, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref) {
        return op(m, "sub", op(m, "mul", x, y), op(m, "div", x, y));
    }, true, {1, 0});
    // a third computed operand while one is saved stays a kernel of its own
    run(16, 64, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref v) {
        auto inner = op(m, "div", op(m, "sub", x, y), op(m, "add", y, bcast(m, v, y)));
        return op(m, "mul", op(m, "add", x, y), inner);
    }, true, {1, 1});
    // longer than one chain may be: split into several
    run(8, 128, [&](module& m, instruction_ref, instruction_ref y, instruction_ref) {
        auto t = y;
        for(int i = 0; i < 20; i++)
            t = op(m, "sqrt", op(m, "add", t, y));
        return t;
    }, true, {4, 0}); // 7 + 7 + 7 + 19 operators
    // an operand whose strides do not reduce to rows and columns keeps the general kernel
    run(64, 64, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref) {
        auto xt = m.add_instruction(make_op("transpose", {{"permutation", {1, 0}}}), x);
        return op(m, "mul", op(m, "add", xt, y), y);
    }, true, {0, 2});
    // a row length that is no multiple of four, and a view that starts off a 16-byte boundary
    run(9, 203, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref) {
        return op(m, "mul", op(m, "sub", x, y), y);
    }, true, {1, 0});
    run(9, 204, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref) {
        auto xs = m.add_instruction(make_op("slice", {{"axes", {1}}, {"starts", {1}}, {"ends", {201}}}), x);
        auto ys = m.add_instruction(make_op("slice", {{"axes", {1}}, {"starts", {4}}, {"ends", {204}}}), y);
        return op(m, "mul", op(m, "sub", xs, ys), ys);
    }, true, {1, 0});
    // GELU as the exporters write it: x * 0.5 * (1 + erf(x / sqrt 2)) after a bias
    run(33, 200, [&](module& m, instruction_ref x, instruction_ref, instruction_ref v) {
        auto constant = [&](float c) {
            return bcast(m, m.add_literal(literal{shape{shape::float_type, {1}}, std::vector<float>{c}}), x);
        };
        auto h = op(m, "add", x, bcast(m, v, x));
        auto e = op(m, "add", op(m, "erf", op(m, "mul", h, constant(0.70710678f))), constant(1.0f));
        return op(m, "mul", op(m, "mul", h, constant(0.5f)), e);
    }, false, {1, 0}); // x + bias has two users: both compute it again, the sum is never stored
    // layer normalisation with its scale and shift: one kernel that holds the row (the means are
    // steps of its chain), equal to the separate operators bit for bit
    run(33, 200, [&](module& m, instruction_ref x, instruction_ref, instruction_ref v) {
        auto mean  = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), x);
        auto xm    = op(m, "sub", x, bcast(m, mean, x));
        auto var   = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), op(m, "mul", xm, xm));
        auto eps   = m.add_literal(literal{shape{shape::float_type, {1}}, std::vector<float>{1e-5f}});
        auto sigma = op(m, "sqrt", op(m, "add", var, bcast(m, eps, var)));
        return op(m, "add", op(m, "mul", op(m, "div", xm, bcast(m, sigma, x)), bcast(m, v, x)), bcast(m, v, x));
    }, false, {0, 0, 1});
    // the form with rsqrt, behind a residual sum that nobody else reads, a tanh behind the shift
    run(130, 768, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref v) {
        auto sum  = op(m, "add", x, y);
        auto mean = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), sum);
        auto d    = op(m, "sub", sum, bcast(m, mean, sum));
        auto var  = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), op(m, "mul", d, d));
        auto eps  = m.add_literal(literal{shape{shape::float_type, {1}}, std::vector<float>{1e-5f}});
        auto rs   = op(m, "rsqrt", op(m, "add", bcast(m, eps, var), var));
        auto n    = op(m, "mul", bcast(m, rs, sum), d);
        return op(m, "tanh", op(m, "add", op(m, "mul", n, bcast(m, v, sum)), y));
    }, false, {0, 0, 1});
    // a residual sum that is read again later is stored by its own operator and read by the kernel;
    // x - mean with a third reader keeps the separate operators
    run(9, 1000, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref) {
        auto sum  = op(m, "add", x, y);
        auto mean = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), sum);
        auto d    = op(m, "sub", sum, bcast(m, mean, sum));
        auto var  = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), op(m, "mul", d, d));
        auto eps  = m.add_literal(literal{shape{shape::float_type, {1}}, std::vector<float>{1e-5f}});
        auto rs   = op(m, "rsqrt", op(m, "add", var, bcast(m, eps, var)));
        return op(m, "add", op(m, "mul", d, bcast(m, rs, sum)), sum);
    }, false, {0, 1, 1});
    run(9, 64, [&](module& m, instruction_ref x, instruction_ref, instruction_ref) {
        auto mean = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), x);
        auto d    = op(m, "sub", x, bcast(m, mean, x));
        auto var  = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), op(m, "mul", d, d));
        auto eps  = m.add_literal(literal{shape{shape::float_type, {1}}, std::vector<float>{1e-5f}});
        auto rs   = op(m, "rsqrt", op(m, "add", var, bcast(m, eps, var)));
        return op(m, "add", op(m, "mul", d, bcast(m, rs, x)), op(m, "neg", d));
    }, false, {2, 2, 0});
    // a value with a user that is no pointwise operator is stored once and read by the others
    run(16, 64, [&](module& m, instruction_ref x, instruction_ref y, instruction_ref) {
        auto d  = op(m, "sub", x, y);
        auto mu = m.add_instruction(make_op("reduce_mean", {{"axes", {-1}}}), d);
        return op(m, "mul", op(m, "add", d, y), bcast(m, mu, x));
    }, false, {1, 1});
}

// agreement of two float tensors as the reference's verify does it (verify.hpp:175-195): root mean
// square of the difference against the root mean square of the expected values
static double rms_error(const argument& got, const argument& want)
{
    auto a = got.to_vector<double>();
    auto b = want.to_vector<double>();
    double num = 0, den = 0;
    for(std::size_t i = 0; i < a.size(); i++)
    {
        num += (a[i] - b[i]) * (a[i] - b[i]);
        den += b[i] * b[i];
    }
    return std::sqrt(num / den);
}

TEST_CASE(encoder_int8_qdq)
{
    // benchmark config 5 at a size the CPU oracle evaluates in seconds: 2 layers, hidden 128, 4 heads,
    // FFN 512, batch 2 x seq 16, vocabulary 100.  Activation scales come from max-abs calibration of
    // the float graph on the seeded input.  The device's erf / exp differ from the host's in the
    // last place and a quantizelinear input that lands within that distance of a rounding boundary
    // moves one int8 step, so the end-to-end outputs are compared by RMS error (1e-3) rather than
    // bit by bit.
    encoder::config c;
    auto w = encoder::make_weights(c, 7);
    argument ids{shape{shape::int32_type, {c.tokens()}}, uniform_ints<int>(c.tokens(), 0, static_cast<int>(c.vocab) - 1, 8)};
    auto scales_cpu = encoder::calibrate(c, w, "oracle", ids);
    auto scales_gpu = encoder::calibrate(c, w, "mi355", ids);
    EXPECT(scales_cpu.size() == 4 * c.layers);
    for(std::size_t i = 0; i < scales_cpu.size(); i++)
        EXPECT(std::fabs(scales_cpu[i] - scales_gpu[i]) <= 1e-5 * scales_cpu[i]);
    auto p = encoder::quantized(c, w, scales_cpu);
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    EXPECT(count_ops(*p.get_main_module(), "quant_dot") == 6 * c.layers);
    EXPECT(count_ops(*p.get_main_module(), "dot") == 2 * c.layers); // the attention products
    auto want = run_on("oracle", p, {{"ids", ids}});
    auto got  = run_on("mi355", p, {{"ids", ids}});
    EXPECT(got[0].get_shape() == shape{shape::float_type, {c.tokens(), c.hidden}});
    const double err = rms_error(got[0], want[0]);
    std::cout << "encoder rms error " << err << std::endl;
    EXPECT(err < 1e-3);
    // every QDQ MatMul became one fused kernel launch
    program compiled = p;
    compiled.compile(migraphx::make_target("mi355"));
    EXPECT(count_ops(*compiled.get_main_module(), "mi355::quant_dot") == 6 * c.layers);
    // four quantized activations per layer; the GELU's, which nothing else reads, is quantized by the
    // chain that computes it
    EXPECT(count_ops(*compiled.get_main_module(), "mi355::quantizelinear") == 3 * c.layers);
    EXPECT(count_ops(*compiled.get_main_module(), "mi355::chain_q8") == c.layers);
    // each layer normalisation (one behind the embeddings, two per layer) is one kernel, the residual
    // sum in front of it included
    EXPECT(count_ops(*compiled.get_main_module(), "mi355::chain_rows") == 2 * c.layers + 1);
    EXPECT(not has_op(compiled, "mi355::reduce_mean"));
    EXPECT(not has_op(compiled, "mi355::dequantizelinear"));
    // and the quantized model stays close to the float one
    encoder::builder fb{c, w, {}, {}};
    fb.tap = [](std::size_t, std::vector<argument>) {};
    auto fp = fb.build();
    auto ref = run_on("oracle", fp, {{"ids", ids}});
    EXPECT(rms_error(want[0], ref[0]) < 0.05);
}

TEST_CASE(compiled_program_saved_and_loaded)
{
    // A program compiled for the device (fused quant_dot launches, device literals holding the
    // folded int8 weights and column sums, scratch allocations, copies inside eval) is written to
    // a file, read back in the same process and run: same instructions, bit-identical results
    // (test/serialize_program.cpp:88-95, on this target).
    encoder::config c;
    auto w = encoder::make_weights(c, 7);
    argument ids{shape{shape::int32_type, {c.tokens()}}, uniform_ints<int>(c.tokens(), 0, static_cast<int>(c.vocab) - 1, 8)};
    auto scales = encoder::calibrate(c, w, "mi355", ids);
    auto p      = encoder::quantized(c, w, scales);
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    program compiled = p;
    migraphx::compile_options opts;
    opts.offload_copy = true;
    compiled.compile(migraphx::make_target("mi355"), opts);
    auto want = compiled.eval({{"ids", ids}});
    compiled.finish();

    const std::string filename = "/tmp/mi355_gpu_tests_encoder.mxr";
    migraphx::save(compiled, filename);
    auto loaded = migraphx::load(filename);
    std::remove(filename.c_str());
    EXPECT(loaded.is_compiled());
    EXPECT(loaded == compiled);
    EXPECT(count_ops(*loaded.get_main_module(), "mi355::quant_dot") == 6 * c.layers);
    EXPECT(count_ops(*loaded.get_main_module(), "mi355::literal") ==
           count_ops(*compiled.get_main_module(), "mi355::literal"));
    for(int rep = 0; rep < 2; rep++)
    {
        auto got = loaded.eval({{"ids", ids}});
        loaded.finish();
        EXPECT(got.size() == 1 and same_bytes(got[0], want[0]));
    }
    // the JSON form carries the same program
    migraphx::file_options json;
    json.format  = "json";
    auto loaded2 = migraphx::load_buffer(migraphx::save_buffer(compiled, json), json);
    auto got2    = loaded2.eval({{"ids", ids}});
    loaded2.finish();
    EXPECT(same_bytes(got2[0], want[0]));

    // weight-only int4: the packed weights and their scales travel as device literals
    {
        const std::size_t m = 4, k = 256, n = 192;
        program q;
        auto* mm = q.get_main_module();
        auto x   = mm->add_parameter("x", shape{shape::half_type, {m, k}});
        auto wl  = mm->add_literal(literal{shape{shape::half_type, {k, n}}, normal_floats(k * n, 0.05f, 21)});
        mm->add_return({mm->add_instruction(make_op("dot"), x, wl)});
        migraphx::quantize_int4_weights(q);
        program cq = q;
        cq.compile(migraphx::make_target("mi355"), opts);
        argument xa{shape{shape::half_type, {m, k}}, normal_floats(m * k, 1.0f, 22)};
        auto r1 = cq.eval({{"x", xa}});
        cq.finish();
        auto lq = migraphx::load_buffer(migraphx::save_buffer(cq));
        auto r2 = lq.eval({{"x", xa}});
        lq.finish();
        EXPECT(lq == cq);
        EXPECT(same_bytes(r1[0], r2[0]));
    }
}

TEST_CASE(encoder_int8_qdq_real_width)
{
    // benchmark config 5 at its real layer width -- hidden 768, 12 heads of 64, FFN 3072, sequence
    // 384, vocabulary 30522 -- for two layers and one sequence, which the CPU oracle still evaluates
    // in seconds: the shapes every one of the 72 quantized MatMuls and 24 attention products of the
    // full model has.  Same comparison as the small model (RMS 1e-3 against the CPU target) with the
    // float `dot`s reproducing the reference's double sum.  With the `dot`s on the fp32 matrix cores
    // (MIGRAPHX_MI355_FP32_DOT) the attention outputs move in their last bits, which is enough to
    // carry some inputs of the following quantizelinear across a rounding boundary: each such
    // input moves one int8 step (0.8 % of the tensor's range), and the end-to-end RMS error comes
    // out at 1.4e-3 -- outside the 1e-3 the default mode meets, which is why the mode is opt-in.
    // It is held to 3e-3 here.
    encoder::config c;
    c.layers = 2;
    c.hidden = 768;
    c.heads  = 12;
    c.ffn    = 3072;
    c.batch  = 1;
    c.seq    = 384;
    c.vocab  = 30522;
    auto w   = encoder::make_weights(c, 17);
    argument ids{shape{shape::int32_type, {c.tokens()}}, uniform_ints<int>(c.tokens(), 0, static_cast<int>(c.vocab) - 1, 18)};
    auto scales = encoder::calibrate(c, w, "mi355", ids);
    auto p      = encoder::quantized(c, w, scales);
    migraphx::run_passes(p, {migraphx::simplify_qdq{}, migraphx::dead_code_elimination{}});
    EXPECT(count_ops(*p.get_main_module(), "quant_dot") == 6 * c.layers);
    auto want = run_on("oracle", p, {{"ids", ids}});
    auto got  = run_on("mi355", p, {{"ids", ids}});
    const double err = rms_error(got[0], want[0]);
    std::cout << "real-width encoder rms error, exact float dots " << err << std::endl;
    EXPECT(err < 1e-3);
    setenv("MIGRAPHX_MI355_FP32_DOT", "1", 1);
    auto fast = run_on("mi355", p, {{"ids", ids}});
    program compiled = p;
    compiled.compile(migraphx::make_target("mi355"));
    unsetenv("MIGRAPHX_MI355_FP32_DOT");
    const double err32 = rms_error(fast[0], want[0]);
    std::cout << "real-width encoder rms error, fp32 float dots " << err32 << std::endl;
    EXPECT(err32 < 3e-3);
    std::size_t fast_dots = 0;
    for(auto ins = compiled.get_main_module()->begin(); ins != compiled.get_main_module()->end(); ++ins)
        if(ins->name() == "mi355::dot" and ins->get_operator().to_value().at("fp32acc").to<bool>())
            fast_dots++;
    EXPECT(fast_dots == 2 * c.layers);
}

TEST_CASE(encoder_int8_qdq_full_size_replicated)
{
    // benchmark config 5 at its full size -- 12 layers, hidden 768, 12 heads, FFN 3072, 32 sequences
    // of 384 tokens -- which the CPU oracle cannot evaluate in test time.  Every operator of the graph
    // treats the sequences of a batch independently (the MatMuls row by row, attention per sequence and
    // head, LayerNorm / softmax per row), the int8 sums are exact and the float `dot`s add in the
    // reference's order whatever the batch, so a batch of 32 copies of one sequence must give 32 copies,
    // bit for bit, of what the same 12 layers give for that sequence alone -- although the batch takes
    // other kernels (M = 12288 instead of 384: other tiles, no split of K).  The one-sequence program is
    // the shape that `encoder_int8_qdq_real_width` pins against the CPU target layer by layer.
    encoder::config c1;
    c1.layers = 12;
    c1.hidden = 768;
    c1.heads  = 12;
    c1.ffn    = 3072;
    c1.batch  = 1;
    c1.seq    = 384;
    c1.vocab  = 30522;
    encoder::config c32 = c1;
    c32.batch           = 32;
    auto w              = encoder::make_weights(c1, 31);
    auto one            = uniform_ints<int>(c1.tokens(), 0, static_cast<int>(c1.vocab) - 1, 32);
    std::vector<int> many;
    for(std::size_t b = 0; b < c32.batch; b++)
        many.insert(many.end(), one.begin(), one.end());
    argument ids1{shape{shape::int32_type, {c1.tokens()}}, one};
    argument ids32{shape{shape::int32_type, {c32.tokens()}}, many};
    auto scales = encoder::calibrate(c1, w, "mi355", ids1);
    // max-abs calibration sees the same values 32 times over: the same scales
    EXPECT(encoder::calibrate(c32, w, "mi355", ids32) == scales);
    auto p1  = encoder::quantized(c1, w, scales);
    auto p32 = encoder::quantized(c32, w, scales);
    program compiled = p32;
    compiled.compile(migraphx::make_target("mi355"));
    // the q / k / v projections of a layer share their activations: one batched launch, then the
    // output projection and the two feed-forward products
    EXPECT(count_ops(*compiled.get_main_module(), "mi355::quant_dot") == 4 * c32.layers);
    auto alone = run_on("mi355", p1, {{"ids", ids1}})[0];
    auto batch = run_on("mi355", p32, {{"ids", ids32}})[0];
    const std::size_t bytes = alone.get_shape().bytes();
    EXPECT(batch.get_shape().bytes() == bytes * c32.batch);
    std::size_t differing = 0;
    for(std::size_t b = 0; b < c32.batch; b++)
        if(std::memcmp(batch.data() + b * bytes, alone.data(), bytes) != 0)
            differing++;
    EXPECT(differing == 0);
    auto v = alone.to_vector<float>();
    double s = 0;
    for(float f : v)
        s += std::fabs(f);
    EXPECT(std::isfinite(s) and s / v.size() > 0.1);   // LayerNorm output: mean |x| is about 0.8
}

// `gpu_tests encoder_bench [layers]`: the full BERT-base shape (hidden 768, 12 heads, FFN 3072, batch
// 32 x seq 384 = 12288 tokens, vocabulary 30522) on the device: calibration, compile, timed forwards
static int encoder_bench(int argc, char** argv)
{
    encoder::config c;
    c.layers = argc > 2 ? std::atoi(argv[2]) : 12;
    c.hidden = 768;
    c.heads  = 12;
    c.ffn    = 3072;
    c.batch  = 32;
    c.seq    = 384;
    c.vocab  = 30522;
    auto w   = encoder::make_weights(c, 1);
    argument ids{shape{shape::int32_type, {c.tokens()}}, uniform_ints<int>(c.tokens(), 0, 30521, 2)};
    auto t      = migraphx::make_target("mi355");
    auto scales = encoder::calibrate(c, w, "mi355", ids);
    auto p      = encoder::quantized(c, w, scales);
    p.compile(t);
    std::cout << "quantized MatMul launches per forward: "
              << count_ops(*p.get_main_module(), "mi355::quant_dot") << std::endl;
    {
        std::size_t arena = 0, separate = 0, buffers = 0;
        for(auto ins = p.get_main_module()->begin(); ins != p.get_main_module()->end(); ++ins)
        {
            if(ins->name() == "mi355::arena")
                arena = ins->get_shape().bytes();
            if(ins->name() == "mi355::load" or ins->name() == "mi355::allocate")
            {
                separate += ins->get_shape().bytes();
                buffers++;
            }
        }
        std::cout << "intermediate buffers: " << buffers << " of " << separate / 1048576.0 << " MiB in all, arena "
                  << arena / 1048576.0 << " MiB" << std::endl;
    }
    auto dids = t.copy_to(ids);
    for(int i = 0; i < 2; i++)
        p.eval({{"ids", dids}});
    p.finish();
    const int iters = 5;
    auto t0 = std::chrono::steady_clock::now();
    for(int i = 0; i < iters; i++)
        p.eval({{"ids", dids}});
    p.finish();
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / iters;
    const double gemm_ops = 2.0 * c.tokens() * c.layers * (4.0 * c.hidden * c.hidden + 2.0 * c.hidden * c.ffn);
    std::cout << "layers " << c.layers << ": " << ms << " ms per forward, quantized MatMuls "
              << gemm_ops / 1e12 << " TOP -> " << gemm_ops / (ms * 1e9) << " TOPS if they were all of it" << std::endl;
    auto out = t.copy_from(p.eval({{"ids", dids}})[0]).to_vector<float>();
    double s = 0;
    for(float v : out)
        s += std::fabs(v);
    std::cout << "mean |output| " << s / out.size() << std::endl;
    return std::isfinite(s) ? 0 : 1;
}

int main(int argc, char** argv)
{
    try
    {
        if(argc > 1 and std::string(argv[1]) == "encoder_bench")
            return encoder_bench(argc, argv);
        return test::run(argc, argv);
    }
    catch(const std::exception& e)
    {
        std::cout << "error: " << e.what() << std::endl;
        return 4;
    }
}
