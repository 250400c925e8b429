/* The C interface (include/migraphx/migraphx.h) driven from C, the way the reference's
 * tests under test/api/ drive theirs: a QDQ matmul is built instruction by instruction, quantized, saved,
 * loaded, compiled and run; an ONNX file is parsed with input-shape options; error statuses are
 * checked.  argv[1] names the target ("oracle", the test programs' CPU target, by default; "gpu"
 * for the device).  Compiled as C so that the header is known to be C-clean.
 */
#include <migraphx/migraphx.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static int failures = 0;
#define CHECK(cond)                                                          \
    do                                                                       \
    {                                                                        \
        if(!(cond))                                                          \
        {                                                                    \
            printf("%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
            failures++;                                                      \
        }                                                                    \
    } while(0)
#define OK(call) CHECK((call) == migraphx_status_success)

static migraphx_instruction_t
add(migraphx_module_t m, const char* op_name, const char* attrs, migraphx_instruction_t* in, size_t n)
{
    migraphx_operation_t op;
    migraphx_instructions_t args;
    migraphx_instruction_t out = NULL;
    OK(migraphx_operation_create(&op, op_name, attrs));
    OK(migraphx_instructions_create(&args, (const const_migraphx_instruction_t*)in, n));
    OK(migraphx_module_add_instruction(&out, m, op, args));
    OK(migraphx_instructions_destroy(args));
    OK(migraphx_operation_destroy(op));
    return out;
}

static void test_shapes(void)
{
    size_t lens[3] = {2, 3, 4};
    size_t strides[3] = {12, 1, 3};
    migraphx_shape_t s, t, u;
    OK(migraphx_shape_create(&s, migraphx_shape_half_type, lens, 3));
    OK(migraphx_shape_create_with_strides(&t, migraphx_shape_half_type, lens, 3, strides, 3));
    OK(migraphx_shape_create_scalar(&u, migraphx_shape_int8_type));
    const size_t* out;
    size_t n, v;
    bool b;
    migraphx_shape_datatype_t dt;
    OK(migraphx_shape_lengths(&out, &n, s));
    CHECK(n == 3 && out[0] == 2 && out[1] == 3 && out[2] == 4);
    OK(migraphx_shape_strides(&out, &n, s));
    CHECK(n == 3 && out[0] == 12 && out[1] == 4 && out[2] == 1);
    OK(migraphx_shape_type(&dt, s));
    CHECK(dt == migraphx_shape_half_type);
    OK(migraphx_shape_elements(&v, s));
    CHECK(v == 24);
    OK(migraphx_shape_bytes(&v, s));
    CHECK(v == 48);
    OK(migraphx_shape_ndim(&v, s));
    CHECK(v == 3);
    OK(migraphx_shape_standard(&b, s));
    CHECK(b);
    OK(migraphx_shape_standard(&b, t));
    CHECK(!b);
    OK(migraphx_shape_dynamic(&b, t));
    CHECK(!b);
    OK(migraphx_shape_equal(&b, s, t));
    CHECK(!b);
    OK(migraphx_shape_index(&v, t, 5)); /* element (0, 1, 1) */
    CHECK(v == 1 + 3);
    OK(migraphx_shape_assign_to(t, s));
    OK(migraphx_shape_equal(&b, s, t));
    CHECK(b);
    OK(migraphx_shape_type(&dt, u));
    CHECK(dt == migraphx_shape_int8_type);
    /* every element type keeps the reference's number through a round trip */
    for(int k = migraphx_shape_bool_type; k <= migraphx_shape_fp8e5m2fnuz_type; k++)
    {
        migraphx_shape_t x;
        OK(migraphx_shape_create_scalar(&x, (migraphx_shape_datatype_t)k));
        OK(migraphx_shape_type(&dt, x));
        CHECK((int)dt == k);
        OK(migraphx_shape_destroy(x));
    }
    CHECK(migraphx_shape_create(NULL, migraphx_shape_float_type, lens, 3) == migraphx_status_bad_param);
    CHECK(migraphx_shape_create_scalar(&u, (migraphx_shape_datatype_t)77) == migraphx_status_bad_param);
    CHECK(migraphx_shape_elements(&v, NULL) == migraphx_status_bad_param);
    OK(migraphx_shape_destroy(s));
    OK(migraphx_shape_destroy(t));
}

static void test_arguments(void)
{
    size_t lens[2] = {3, 5};
    migraphx_shape_t s;
    OK(migraphx_shape_create(&s, migraphx_shape_float_type, lens, 2));
    float data[15];
    for(int i = 0; i < 15; i++)
        data[i] = (float)i * 0.5f;
    migraphx_argument_t a, e, g1, g2, l;
    OK(migraphx_argument_create(&a, s, data)); /* a view */
    char* buf;
    OK(migraphx_argument_buffer(&buf, a));
    CHECK(buf == (char*)data);
    const_migraphx_shape_t as;
    OK(migraphx_argument_shape(&as, a));
    bool b;
    OK(migraphx_shape_equal(&b, as, s));
    CHECK(b);
    OK(migraphx_argument_create_empty(&e, s));
    OK(migraphx_argument_buffer(&buf, e));
    CHECK(buf != NULL && buf != (char*)data);
    memcpy(buf, data, sizeof(data));
    OK(migraphx_argument_equal(&b, a, e));
    CHECK(b);
    buf[0] = 1;
    OK(migraphx_argument_equal(&b, a, e));
    CHECK(!b);
    /* generated data repeats for a seed, differs between seeds, and stays in [-1, 1) */
    OK(migraphx_argument_generate(&g1, s, 3));
    OK(migraphx_argument_generate(&g2, s, 3));
    OK(migraphx_argument_equal(&b, g1, g2));
    CHECK(b);
    OK(migraphx_argument_destroy(g2));
    OK(migraphx_argument_generate(&g2, s, 4));
    OK(migraphx_argument_equal(&b, g1, g2));
    CHECK(!b);
    OK(migraphx_argument_buffer(&buf, g1));
    for(int i = 0; i < 15; i++)
    {
        const float x = ((float*)buf)[i];
        CHECK(x >= -1.0f && x < 1.0f && x * 16.0f == floorf(x * 16.0f));
    }
    /* to a file and back */
    OK(migraphx_argument_save(a, "/tmp/mi355_capi_argument.msgpack"));
    OK(migraphx_argument_load(&l, "/tmp/mi355_capi_argument.msgpack"));
    remove("/tmp/mi355_capi_argument.msgpack");
    OK(migraphx_argument_equal(&b, a, l));
    CHECK(b);
    CHECK(migraphx_argument_load(&l, "/tmp/mi355_capi_no_such_file") == migraphx_status_unknown_error);
    OK(migraphx_argument_destroy(a));
    OK(migraphx_argument_destroy(e));
    OK(migraphx_argument_destroy(g1));
    OK(migraphx_argument_destroy(g2));
    OK(migraphx_argument_destroy(l));
    OK(migraphx_shape_destroy(s));
}

static void test_operations(void)
{
    migraphx_operation_t op;
    char name[64];
    OK(migraphx_operation_create(&op, "transpose", "{permutation: [%d, %d]}", 1, 0));
    OK(migraphx_operation_name(name, sizeof(name), op));
    CHECK(strcmp(name, "transpose") == 0);
    OK(migraphx_operation_name(name, 4, op)); /* truncated, still terminated */
    CHECK(strcmp(name, "tra") == 0);
    OK(migraphx_operation_destroy(op));
    OK(migraphx_operation_create(&op, "slice", "axes: [1], starts: [0], \"ends\": [2]")); /* braces optional */
    OK(migraphx_operation_destroy(op));
    OK(migraphx_operation_create(&op, "dot", NULL));
    OK(migraphx_operation_destroy(op));
    CHECK(migraphx_operation_create(&op, "no_such_operator", NULL) == migraphx_status_unknown_error);
    CHECK(migraphx_operation_create(&op, "transpose", "{no_such_attribute: 1}") == migraphx_status_unknown_error);
    CHECK(migraphx_operation_create(&op, "transpose", "{permutation: [1, }") == migraphx_status_unknown_error);
    CHECK(migraphx_operation_create(NULL, "dot", NULL) == migraphx_status_bad_param);
}

/* x[m, k] (float parameter) -> quantizelinear -> dequantizelinear -> dot with dequantized int8
 * weights [k, n]; returns the program and fills `want` with the float product of the dequantized
 * operands, which every value here represents exactly */
#define M 4
#define K 8
#define N 6
static migraphx_program_t build_qdq_matmul(float* x, float* want)
{
    migraphx_program_t p;
    migraphx_module_t mm;
    OK(migraphx_program_create(&p));
    OK(migraphx_program_get_main_module(&mm, p));
    size_t xl[2] = {M, K}, wl[2] = {K, N};
    migraphx_shape_t xs, ws, fs, is;
    OK(migraphx_shape_create(&xs, migraphx_shape_float_type, xl, 2));
    OK(migraphx_shape_create(&ws, migraphx_shape_int8_type, wl, 2));
    OK(migraphx_shape_create_scalar(&fs, migraphx_shape_float_type));
    OK(migraphx_shape_create_scalar(&is, migraphx_shape_int8_type));
    int8_t w[K * N];
    for(int i = 0; i < K * N; i++)
        w[i] = (int8_t)((i * 7) % 23 - 11);
    for(int i = 0; i < M * K; i++)
        x[i] = 0.25f * (float)((i * 5) % 17 - 8); /* multiples of the activation scale */
    const float sx = 0.25f, sw = 0.5f;
    const int8_t zero = 0;
    migraphx_instruction_t px, lw, lsx, lsw, lz;
    OK(migraphx_module_add_parameter(&px, mm, "x", xs));
    OK(migraphx_module_add_literal(&lw, mm, ws, (const char*)w));
    OK(migraphx_module_add_literal(&lsx, mm, fs, (const char*)&sx));
    OK(migraphx_module_add_literal(&lsw, mm, fs, (const char*)&sw));
    OK(migraphx_module_add_literal(&lz, mm, is, (const char*)&zero));
    migraphx_instruction_t in[3];
    in[0] = lsx;
    migraphx_instruction_t bsx = add(mm, "multibroadcast", "{out_lens: [4, 8]}", in, 1);
    in[0] = lz;
    migraphx_instruction_t bzx = add(mm, "multibroadcast", "{out_lens: [4, 8]}", in, 1);
    in[0] = lsw;
    migraphx_instruction_t bsw = add(mm, "multibroadcast", "{out_lens: [8, 6]}", in, 1);
    in[0] = lz;
    migraphx_instruction_t bzw = add(mm, "multibroadcast", "{out_lens: [8, 6]}", in, 1);
    in[0] = px, in[1] = bsx, in[2] = bzx;
    migraphx_instruction_t q = add(mm, "quantizelinear", NULL, in, 3);
    in[0] = q;
    migraphx_instruction_t dq = add(mm, "dequantizelinear", NULL, in, 3);
    in[0] = lw, in[1] = bsw, in[2] = bzw;
    migraphx_instruction_t dw = add(mm, "dequantizelinear", NULL, in, 3);
    in[0] = dq, in[1] = dw;
    migraphx_instruction_t d = add(mm, "dot", NULL, in, 2);
    migraphx_instructions_t rets;
    migraphx_instruction_t r;
    OK(migraphx_instructions_create(&rets, (const const_migraphx_instruction_t*)&d, 1));
    OK(migraphx_module_add_return(&r, mm, rets));
    OK(migraphx_instructions_destroy(rets));
    for(int i = 0; i < M; i++)
        for(int j = 0; j < N; j++)
        {
            float acc = 0;
            for(int kk = 0; kk < K; kk++)
                acc += x[i * K + kk] * (sw * (float)w[kk * N + j]);
            want[i * N + j] = acc;
        }
    migraphx_instruction_t all[] = {px, lw, lsx, lsw, lz, bsx, bzx, bsw, bzw, q, dq, dw, d, r};
    for(size_t i = 0; i < sizeof(all) / sizeof(all[0]); i++)
        OK(migraphx_instruction_destroy(all[i]));
    OK(migraphx_shape_destroy(xs));
    OK(migraphx_shape_destroy(ws));
    OK(migraphx_shape_destroy(fs));
    OK(migraphx_shape_destroy(is));
    return p;
}

static void run_and_check(migraphx_program_t p, float* x, const float* want, const char* what)
{
    migraphx_program_parameter_shapes_t pshapes;
    OK(migraphx_program_get_parameter_shapes(&pshapes, p));
    size_t n;
    OK(migraphx_program_parameter_shapes_size(&n, pshapes));
    CHECK(n == 1);
    const char* names[1] = {NULL};
    OK(migraphx_program_parameter_shapes_names(names, pshapes));
    CHECK(names[0] != NULL && strcmp(names[0], "x") == 0);
    const_migraphx_shape_t xs;
    OK(migraphx_program_parameter_shapes_get(&xs, pshapes, "x"));
    CHECK(migraphx_program_parameter_shapes_get(&xs, pshapes, "y") == migraphx_status_bad_param);
    OK(migraphx_program_parameter_shapes_get(&xs, pshapes, "x"));
    migraphx_argument_t xa;
    OK(migraphx_argument_create(&xa, xs, x));
    migraphx_program_parameters_t params;
    OK(migraphx_program_parameters_create(&params));
    OK(migraphx_program_parameters_add(params, "x", xa));
    migraphx_arguments_t results;
    OK(migraphx_program_run(&results, p, params));
    OK(migraphx_arguments_size(&n, results));
    CHECK(n == 1);
    const_migraphx_argument_t r0;
    OK(migraphx_arguments_get(&r0, results, 0));
    CHECK(migraphx_arguments_get(&r0, results, 1) == migraphx_status_bad_param);
    OK(migraphx_arguments_get(&r0, results, 0));
    const_migraphx_shape_t rs;
    OK(migraphx_argument_shape(&rs, r0));
    const size_t* lens;
    OK(migraphx_shape_lengths(&lens, &n, rs));
    CHECK(n == 2 && lens[0] == M && lens[1] == N);
    char* buf;
    OK(migraphx_argument_buffer(&buf, r0));
    int wrong = 0;
    for(int i = 0; i < M * N; i++)
        wrong += ((float*)buf)[i] != want[i];
    if(wrong != 0)
        printf("%s: %d of %d results differ\n", what, wrong, M * N);
    CHECK(wrong == 0);
    /* a parameter that is missing is an error, not a crash */
    migraphx_program_parameters_t none;
    migraphx_arguments_t unused;
    OK(migraphx_program_parameters_create(&none));
    CHECK(migraphx_program_run(&unused, p, none) == migraphx_status_unknown_error);
    OK(migraphx_program_parameters_destroy(none));
    migraphx_context_t ctx;
    OK(migraphx_program_experimental_get_context(&ctx, p));
    OK(migraphx_context_finish(ctx));
    OK(migraphx_arguments_destroy(results));
    OK(migraphx_program_parameters_destroy(params));
    OK(migraphx_argument_destroy(xa));
    OK(migraphx_program_parameter_shapes_destroy(pshapes));
}

static void test_program(const char* target_name)
{
    float x[M * K], want[M * N];
    migraphx_program_t p = build_qdq_matmul(x, want);
    migraphx_shapes_t outs;
    size_t n;
    OK(migraphx_program_get_output_shapes(&outs, p));
    OK(migraphx_shapes_size(&n, outs));
    CHECK(n == 1);
    const_migraphx_shape_t o0;
    OK(migraphx_shapes_get(&o0, outs, 0));
    migraphx_shape_datatype_t dt;
    OK(migraphx_shape_type(&dt, o0));
    CHECK(dt == migraphx_shape_float_type);
    OK(migraphx_shapes_destroy(outs));

    /* saved and loaded before compiling: the same program, in both formats */
    migraphx_file_options_t json;
    OK(migraphx_file_options_create(&json));
    OK(migraphx_file_options_set_file_format(json, "json"));
    migraphx_program_t p2, p3;
    bool same;
    OK(migraphx_save(p, "/tmp/mi355_capi_program.mxr", NULL));
    OK(migraphx_load(&p2, "/tmp/mi355_capi_program.mxr", NULL));
    OK(migraphx_program_equal(&same, p, p2));
    CHECK(same);
    OK(migraphx_save(p, "/tmp/mi355_capi_program.json", json));
    OK(migraphx_load(&p3, "/tmp/mi355_capi_program.json", json));
    OK(migraphx_program_equal(&same, p, p3));
    CHECK(same);
    CHECK(migraphx_load(&p3, "/tmp/mi355_capi_program.json", NULL) == migraphx_status_unknown_error);
    remove("/tmp/mi355_capi_program.json");
    OK(migraphx_file_options_set_file_format(json, "yaml"));
    CHECK(migraphx_save(p, "/tmp/mi355_capi_program.yaml", json) == migraphx_status_unknown_error);

    migraphx_target_t t;
    CHECK(migraphx_target_create(&t, "no_such_target") == migraphx_status_unknown_target);
    OK(migraphx_target_create(&t, target_name));
    migraphx_compile_options_t co;
    OK(migraphx_compile_options_create(&co));
    OK(migraphx_compile_options_set_offload_copy(co, true));
    OK(migraphx_compile_options_set_fast_math(co, false));
    OK(migraphx_compile_options_set_exhaustive_tune_flag(co, false));
    OK(migraphx_program_compile(p, t, co));
    CHECK(migraphx_program_compile(p, t, co) == migraphx_status_unknown_error); /* twice */
    run_and_check(p, x, want, "compiled");

    /* the compiled program through a file */
    migraphx_program_t p4;
    OK(migraphx_save(p, "/tmp/mi355_capi_program.mxr", NULL));
    OK(migraphx_load(&p4, "/tmp/mi355_capi_program.mxr", NULL));
    remove("/tmp/mi355_capi_program.mxr");
    run_and_check(p4, x, want, "compiled, saved, loaded");

    /* the copy loaded earlier compiles and runs on its own */
    OK(migraphx_program_compile(p2, t, co));
    run_and_check(p2, x, want, "loaded, then compiled");
    OK(migraphx_program_assign_to(p3, p2));
    OK(migraphx_program_equal(&same, p3, p2));
    CHECK(same);

    OK(migraphx_compile_options_destroy(co));
    OK(migraphx_target_destroy(t));
    OK(migraphx_file_options_destroy(json));
    OK(migraphx_program_destroy(p));
    OK(migraphx_program_destroy(p2));
    OK(migraphx_program_destroy(p3));
    OK(migraphx_program_destroy(p4));
}

/* a float matmul quantized through the C interface with calibration data: the result stays within
 * int8 quantization error of the float one, and the program holds quantizelinear afterwards */
static void test_quantize(const char* target_name)
{
    migraphx_program_t p;
    migraphx_module_t mm;
    OK(migraphx_program_create(&p));
    OK(migraphx_program_get_main_module(&mm, p));
    size_t xl[2] = {M, 64}, wl[2] = {64, N};
    migraphx_shape_t xs, ws;
    OK(migraphx_shape_create(&xs, migraphx_shape_float_type, xl, 2));
    OK(migraphx_shape_create(&ws, migraphx_shape_float_type, wl, 2));
    migraphx_argument_t xa, wa;
    OK(migraphx_argument_generate(&xa, xs, 1));
    OK(migraphx_argument_generate(&wa, ws, 2));
    char *xb, *wb;
    OK(migraphx_argument_buffer(&xb, xa));
    OK(migraphx_argument_buffer(&wb, wa));
    migraphx_instruction_t px, lw, in[2], d, r;
    OK(migraphx_module_add_parameter(&px, mm, "x", xs));
    OK(migraphx_module_add_literal(&lw, mm, ws, wb));
    in[0] = px, in[1] = lw;
    d = add(mm, "dot", NULL, in, 2);
    migraphx_instructions_t rets;
    OK(migraphx_instructions_create(&rets, (const const_migraphx_instruction_t*)&d, 1));
    OK(migraphx_module_add_return(&r, mm, rets));
    OK(migraphx_instructions_destroy(rets));

    float want[M * N];
    for(int i = 0; i < M; i++)
        for(int j = 0; j < N; j++)
        {
            double acc = 0;
            for(int kk = 0; kk < 64; kk++)
                acc += (double)((float*)xb)[i * 64 + kk] * ((float*)wb)[kk * N + j];
            want[i * N + j] = (float)acc;
        }

    migraphx_target_t t;
    OK(migraphx_target_create(&t, target_name));
    migraphx_program_parameters_t calib;
    OK(migraphx_program_parameters_create(&calib));
    OK(migraphx_program_parameters_add(calib, "x", xa));
    migraphx_quantize_int8_options_t qo;
    OK(migraphx_quantize_int8_options_create(&qo));
    OK(migraphx_quantize_int8_options_add_calibration_data(qo, calib));
    /* only the pair {dot, convolution} is accepted (src/quantization.cpp:181-185) */
    OK(migraphx_quantize_int8_options_add_op_name(qo, "dot"));
    CHECK(migraphx_quantize_int8(p, t, qo) == migraphx_status_unknown_error);
    OK(migraphx_quantize_int8_options_add_op_name(qo, "convolution"));
    OK(migraphx_quantize_int8(p, t, qo));
    migraphx_compile_options_t co;
    OK(migraphx_compile_options_create(&co));
    OK(migraphx_compile_options_set_offload_copy(co, true));
    OK(migraphx_program_compile(p, t, co));
    migraphx_arguments_t results;
    OK(migraphx_program_run(&results, p, calib));
    const_migraphx_argument_t r0;
    OK(migraphx_arguments_get(&r0, results, 0));
    char* buf;
    OK(migraphx_argument_buffer(&buf, r0));
    double worst = 0;
    for(int i = 0; i < M * N; i++)
        worst = fmax(worst, fabs(((float*)buf)[i] - want[i]));
    /* 64 products of values in [-1, 1) quantized to 1/127 steps */
    CHECK(worst < 0.15);
    CHECK(worst > 0.0); /* it was quantized */

    /* fp8 through the same route, on a fresh program */
    migraphx_program_t p8;
    OK(migraphx_program_create(&p8));
    OK(migraphx_program_get_main_module(&mm, p8));
    migraphx_instruction_t px8, lw8, d8, r8;
    OK(migraphx_module_add_parameter(&px8, mm, "x", xs));
    OK(migraphx_module_add_literal(&lw8, mm, ws, wb));
    in[0] = px8, in[1] = lw8;
    d8 = add(mm, "dot", NULL, in, 2);
    OK(migraphx_instructions_create(&rets, (const const_migraphx_instruction_t*)&d8, 1));
    OK(migraphx_module_add_return(&r8, mm, rets));
    OK(migraphx_instructions_destroy(rets));
    migraphx_quantize_fp8_options_t fo;
    OK(migraphx_quantize_fp8_options_create(&fo));
    OK(migraphx_quantize_fp8_options_add_calibration_data(fo, calib));
    OK(migraphx_quantize_fp8(p8, t, fo));
    OK(migraphx_program_compile(p8, t, co));
    migraphx_arguments_t results8;
    OK(migraphx_program_run(&results8, p8, calib));
    OK(migraphx_arguments_get(&r0, results8, 0));
    OK(migraphx_argument_buffer(&buf, r0));
    worst = 0;
    for(int i = 0; i < M * N; i++)
        worst = fmax(worst, fabs(((float*)buf)[i] - want[i]));
    CHECK(worst < 0.6 && worst > 0.0); /* 3 mantissa bits */

    /* weight-only int4 leaves a program that still compiles and runs */
    migraphx_program_t p4;
    OK(migraphx_program_create(&p4));
    OK(migraphx_program_get_main_module(&mm, p4));
    migraphx_instruction_t px4, lw4, d4, r4;
    OK(migraphx_module_add_parameter(&px4, mm, "x", xs));
    OK(migraphx_module_add_literal(&lw4, mm, ws, wb));
    in[0] = px4, in[1] = lw4;
    d4 = add(mm, "dot", NULL, in, 2);
    OK(migraphx_instructions_create(&rets, (const const_migraphx_instruction_t*)&d4, 1));
    OK(migraphx_module_add_return(&r4, mm, rets));
    OK(migraphx_instructions_destroy(rets));
    OK(migraphx_quantize_int4_weights(p4));
    OK(migraphx_program_compile(p4, t, co));
    migraphx_arguments_t results4;
    OK(migraphx_program_run(&results4, p4, calib));
    OK(migraphx_arguments_get(&r0, results4, 0));
    OK(migraphx_argument_buffer(&buf, r0));
    worst = 0;
    for(int i = 0; i < M * N; i++)
        worst = fmax(worst, fabs(((float*)buf)[i] - want[i]));
    CHECK(worst < 2.0 && worst > 0.0); /* one 4-bit grid over the whole weight tensor */

    migraphx_instruction_t all[] = {px, lw, d, r, px8, lw8, d8, r8, px4, lw4, d4, r4};
    for(size_t i = 0; i < sizeof(all) / sizeof(all[0]); i++)
        OK(migraphx_instruction_destroy(all[i]));
    OK(migraphx_arguments_destroy(results));
    OK(migraphx_arguments_destroy(results8));
    OK(migraphx_arguments_destroy(results4));
    OK(migraphx_quantize_int8_options_destroy(qo));
    OK(migraphx_quantize_fp8_options_destroy(fo));
    OK(migraphx_compile_options_destroy(co));
    OK(migraphx_program_parameters_destroy(calib));
    OK(migraphx_target_destroy(t));
    OK(migraphx_program_destroy(p));
    OK(migraphx_program_destroy(p8));
    OK(migraphx_program_destroy(p4));
    OK(migraphx_argument_destroy(xa));
    OK(migraphx_argument_destroy(wa));
    OK(migraphx_shape_destroy(xs));
    OK(migraphx_shape_destroy(ws));
}

/* argv[2]: an ONNX file with one input "x" of shape [batch, 8] (batch symbolic) times an 8 x 4
 * initializer */
static void test_onnx(const char* filename)
{
    FILE* f = fopen(filename, "rb");
    CHECK(f != NULL);
    if(f == NULL)
        return;
    static char data[1 << 16];
    const size_t size = fread(data, 1, sizeof(data), f);
    fclose(f);
    migraphx_program_t p;
    migraphx_program_parameter_shapes_t ps;
    const_migraphx_shape_t xs;
    const size_t* lens;
    size_t n;
    /* default: the open dimension becomes 1 */
    OK(migraphx_parse_onnx(&p, filename, NULL));
    OK(migraphx_program_get_parameter_shapes(&ps, p));
    OK(migraphx_program_parameter_shapes_get(&xs, ps, "x"));
    OK(migraphx_shape_lengths(&lens, &n, xs));
    CHECK(n == 2 && lens[0] == 1 && lens[1] == 8);
    OK(migraphx_program_parameter_shapes_destroy(ps));
    OK(migraphx_program_destroy(p));
    /* default_dim_value */
    migraphx_onnx_options_t o;
    OK(migraphx_onnx_options_create(&o));
    OK(migraphx_onnx_options_set_default_dim_value(o, 3));
    OK(migraphx_parse_onnx_buffer(&p, data, size, o));
    OK(migraphx_program_get_parameter_shapes(&ps, p));
    OK(migraphx_program_parameter_shapes_get(&xs, ps, "x"));
    OK(migraphx_shape_lengths(&lens, &n, xs));
    CHECK(n == 2 && lens[0] == 3 && lens[1] == 8);
    OK(migraphx_program_parameter_shapes_destroy(ps));
    OK(migraphx_program_destroy(p));
    /* an explicit input shape wins */
    size_t dims[2] = {5, 8};
    OK(migraphx_onnx_options_set_input_parameter_shape(o, "x", dims, 2));
    OK(migraphx_parse_onnx_buffer(&p, data, size, o));
    migraphx_shapes_t outs;
    const_migraphx_shape_t o0;
    OK(migraphx_program_get_output_shapes(&outs, p));
    OK(migraphx_shapes_get(&o0, outs, 0));
    OK(migraphx_shape_lengths(&lens, &n, o0));
    CHECK(n == 2 && lens[0] == 5 && lens[1] == 4);
    OK(migraphx_shapes_destroy(outs));
    OK(migraphx_program_destroy(p));
    OK(migraphx_onnx_options_destroy(o));
    CHECK(migraphx_parse_onnx(&p, "/tmp/mi355_capi_no_such.onnx", NULL) == migraphx_status_unknown_error);
    CHECK(migraphx_parse_onnx_buffer(&p, "junk", 4, NULL) == migraphx_status_unknown_error);
}

int main(int argc, char** argv)
{
    const char* target_name = argc > 1 ? argv[1] : "oracle";
    /* the error paths print their messages on stderr; keep the test's own output readable */
    if(getenv("CAPI_TESTS_VERBOSE") == NULL && freopen("/dev/null", "w", stderr) == NULL)
        return 3;
    test_shapes();
    test_arguments();
    test_operations();
    test_program(target_name);
    test_quantize(target_name);
    if(argc > 2)
        test_onnx(argv[2]);
    printf("%s: %d failed checks\n", target_name, failures);
    return failures == 0 ? 0 : 1;
}
