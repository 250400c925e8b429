/* C interface of the host layer: the subset of the reference's C API
 * (src/api/include/migraphx/migraphx.h) that the quantized-GEMM path needs -- shapes, arguments,
 * targets, building a program by hand or from ONNX, quantizing, compiling, running, and programs
 * on disk.  Names, argument order, status codes and the numbering of element types are the
 * reference's, so a caller written against its header compiles against this one for these entry
 * points.  Not part of this build: dynamic shapes, submodules, TensorFlow, custom operators, fp16 /
 * bf16 quantization.
 *
 * Every function returns a status; results come back through the first pointer argument.  Objects
 * made by a *_create, *_get_* that returns a non-const handle of a container type, parse, load or
 * run call belong to the caller, who destroys them.  `const_*` handles returned through an out
 * pointer refer into their container and live as long as it does.  The last error's text is
 * printed on stderr as "<function>: Error: <text>", like the reference does
 * (src/api/api.cpp:60-98).
 */
#ifndef MIGRAPHX_GUARD_C_API_MIGRAPHX_H
#define MIGRAPHX_GUARD_C_API_MIGRAPHX_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#define MIGRAPHX_C_EXPORT __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

typedef enum
{
    migraphx_status_success        = 0,
    migraphx_status_bad_param      = 1,
    migraphx_status_unknown_target = 3,
    migraphx_status_unknown_error  = 4
} migraphx_status;

/* the reference's numbering (migraphx.h:34-74) */
typedef enum
{
    migraphx_shape_tuple_type       = 0,
    migraphx_shape_fp4x2_type       = 1,
    migraphx_shape_bool_type        = 2,
    migraphx_shape_half_type        = 3,
    migraphx_shape_float_type       = 4,
    migraphx_shape_double_type      = 5,
    migraphx_shape_uint8_type       = 6,
    migraphx_shape_int8_type        = 7,
    migraphx_shape_uint16_type      = 8,
    migraphx_shape_int16_type       = 9,
    migraphx_shape_int32_type       = 10,
    migraphx_shape_int64_type       = 11,
    migraphx_shape_uint32_type      = 12,
    migraphx_shape_uint64_type      = 13,
    migraphx_shape_fp8e4m3fnuz_type = 14,
    migraphx_shape_fp8e4m3fn_type   = 15,
    migraphx_shape_fp8e5m2_type     = 16,
    migraphx_shape_bf16_type        = 17,
    migraphx_shape_fp8e5m2fnuz_type = 18
} migraphx_shape_datatype_t;

#define MIGRAPHX_C_HANDLE(name)                 \
    typedef struct migraphx_##name* migraphx_##name##_t; \
    typedef const struct migraphx_##name* const_migraphx_##name##_t

MIGRAPHX_C_HANDLE(shape);
MIGRAPHX_C_HANDLE(argument);
MIGRAPHX_C_HANDLE(target);
MIGRAPHX_C_HANDLE(program_parameter_shapes);
MIGRAPHX_C_HANDLE(program_parameters);
MIGRAPHX_C_HANDLE(arguments);
MIGRAPHX_C_HANDLE(shapes);
MIGRAPHX_C_HANDLE(instruction);
MIGRAPHX_C_HANDLE(instructions);
MIGRAPHX_C_HANDLE(module);
MIGRAPHX_C_HANDLE(program);
MIGRAPHX_C_HANDLE(operation);
MIGRAPHX_C_HANDLE(onnx_options);
MIGRAPHX_C_HANDLE(file_options);
MIGRAPHX_C_HANDLE(compile_options);
MIGRAPHX_C_HANDLE(quantize_int8_options);
MIGRAPHX_C_HANDLE(quantize_fp8_options);
MIGRAPHX_C_HANDLE(context);

/* shape */
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_destroy(migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_assign_to(migraphx_shape_t output,
                                                           const_migraphx_shape_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_create(migraphx_shape_t* shape,
                                                        migraphx_shape_datatype_t type,
                                                        size_t* lengths,
                                                        size_t lengths_size);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_create_with_strides(migraphx_shape_t* shape,
                                                                     migraphx_shape_datatype_t type,
                                                                     size_t* lengths,
                                                                     size_t lengths_size,
                                                                     size_t* strides,
                                                                     size_t strides_size);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_create_scalar(migraphx_shape_t* shape,
                                                               migraphx_shape_datatype_t type);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_lengths(const size_t** out,
                                                         size_t* out_size,
                                                         const_migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_strides(const size_t** out,
                                                         size_t* out_size,
                                                         const_migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_type(migraphx_shape_datatype_t* out,
                                                      const_migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_elements(size_t* out, const_migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_bytes(size_t* out, const_migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_ndim(size_t* out, const_migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_equal(bool* out,
                                                       const_migraphx_shape_t shape,
                                                       const_migraphx_shape_t x);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_standard(bool* out, const_migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_dynamic(bool* out, const_migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shape_index(size_t* out,
                                                       const_migraphx_shape_t shape,
                                                       size_t i);

/* argument: `create` views the caller's buffer, `create_empty` and `generate` own theirs */
MIGRAPHX_C_EXPORT migraphx_status migraphx_argument_destroy(migraphx_argument_t argument);
MIGRAPHX_C_EXPORT migraphx_status migraphx_argument_assign_to(migraphx_argument_t output,
                                                              const_migraphx_argument_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_argument_create(migraphx_argument_t* argument,
                                                           const_migraphx_shape_t shape,
                                                           void* buffer);
MIGRAPHX_C_EXPORT migraphx_status migraphx_argument_create_empty(migraphx_argument_t* argument,
                                                                 const_migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_argument_shape(const_migraphx_shape_t* out,
                                                          const_migraphx_argument_t argument);
MIGRAPHX_C_EXPORT migraphx_status migraphx_argument_buffer(char** out,
                                                           const_migraphx_argument_t argument);
MIGRAPHX_C_EXPORT migraphx_status migraphx_argument_equal(bool* out,
                                                          const_migraphx_argument_t argument,
                                                          const_migraphx_argument_t x);
MIGRAPHX_C_EXPORT migraphx_status migraphx_argument_save(const_migraphx_argument_t a,
                                                         const char* filename);
MIGRAPHX_C_EXPORT migraphx_status migraphx_argument_load(migraphx_argument_t* out,
                                                         const char* filename);
MIGRAPHX_C_EXPORT migraphx_status migraphx_argument_generate(migraphx_argument_t* out,
                                                             const_migraphx_shape_t s,
                                                             size_t seed);

/* target */
MIGRAPHX_C_EXPORT migraphx_status migraphx_target_destroy(migraphx_target_t target);
MIGRAPHX_C_EXPORT migraphx_status migraphx_target_assign_to(migraphx_target_t output,
                                                            const_migraphx_target_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_target_create(migraphx_target_t* target, const char* name);

/* name -> shape of a program's parameters */
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_parameter_shapes_destroy(migraphx_program_parameter_shapes_t program_parameter_shapes);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_parameter_shapes_assign_to(migraphx_program_parameter_shapes_t output,
                                            const_migraphx_program_parameter_shapes_t input);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_parameter_shapes_size(size_t* out,
                                       migraphx_program_parameter_shapes_t program_parameter_shapes);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_parameter_shapes_get(const_migraphx_shape_t* out,
                                      migraphx_program_parameter_shapes_t program_parameter_shapes,
                                      const char* name);
/* fills `out`, an array of _size() pointers */
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_parameter_shapes_names(const char** out,
                                        migraphx_program_parameter_shapes_t program_parameter_shapes);

/* name -> argument to run a program with */
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_parameters_destroy(migraphx_program_parameters_t program_parameters);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_parameters_assign_to(migraphx_program_parameters_t output,
                                      const_migraphx_program_parameters_t input);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_parameters_create(migraphx_program_parameters_t* program_parameters);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_parameters_add(migraphx_program_parameters_t program_parameters,
                                const char* name,
                                const_migraphx_argument_t argument);

/* lists */
MIGRAPHX_C_EXPORT migraphx_status migraphx_arguments_destroy(migraphx_arguments_t arguments);
MIGRAPHX_C_EXPORT migraphx_status migraphx_arguments_assign_to(migraphx_arguments_t output,
                                                               const_migraphx_arguments_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_arguments_size(size_t* out, migraphx_arguments_t arguments);
MIGRAPHX_C_EXPORT migraphx_status migraphx_arguments_get(const_migraphx_argument_t* out,
                                                         migraphx_arguments_t arguments,
                                                         size_t idx);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shapes_destroy(migraphx_shapes_t shapes);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shapes_assign_to(migraphx_shapes_t output,
                                                            const_migraphx_shapes_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shapes_size(size_t* out, migraphx_shapes_t shapes);
MIGRAPHX_C_EXPORT migraphx_status migraphx_shapes_get(const_migraphx_shape_t* out,
                                                      migraphx_shapes_t shapes,
                                                      size_t idx);
MIGRAPHX_C_EXPORT migraphx_status migraphx_instruction_destroy(migraphx_instruction_t instruction);
MIGRAPHX_C_EXPORT migraphx_status migraphx_instruction_assign_to(migraphx_instruction_t output,
                                                                 const_migraphx_instruction_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_instructions_destroy(migraphx_instructions_t instructions);
MIGRAPHX_C_EXPORT migraphx_status migraphx_instructions_assign_to(migraphx_instructions_t output,
                                                                  const_migraphx_instructions_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_instructions_create(migraphx_instructions_t* instructions,
                                                               const const_migraphx_instruction_t* ptr,
                                                               size_t size);

/* module: the handle a program gives out refers into the program */
MIGRAPHX_C_EXPORT migraphx_status migraphx_module_print(const_migraphx_module_t module);
MIGRAPHX_C_EXPORT migraphx_status migraphx_module_add_instruction(migraphx_instruction_t* out,
                                                                  migraphx_module_t module,
                                                                  migraphx_operation_t op,
                                                                  migraphx_instructions_t args);
MIGRAPHX_C_EXPORT migraphx_status migraphx_module_add_literal(migraphx_instruction_t* out,
                                                              migraphx_module_t module,
                                                              const_migraphx_shape_t shape,
                                                              const char* buffer);
MIGRAPHX_C_EXPORT migraphx_status migraphx_module_add_parameter(migraphx_instruction_t* out,
                                                                migraphx_module_t module,
                                                                const char* name,
                                                                const_migraphx_shape_t shape);
MIGRAPHX_C_EXPORT migraphx_status migraphx_module_add_return(migraphx_instruction_t* out,
                                                             migraphx_module_t module,
                                                             migraphx_instructions_t args);

/* program */
MIGRAPHX_C_EXPORT migraphx_status migraphx_program_destroy(migraphx_program_t program);
MIGRAPHX_C_EXPORT migraphx_status migraphx_program_assign_to(migraphx_program_t output,
                                                             const_migraphx_program_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_program_create(migraphx_program_t* program);
MIGRAPHX_C_EXPORT migraphx_status migraphx_program_get_main_module(migraphx_module_t* out,
                                                                   migraphx_program_t program);
MIGRAPHX_C_EXPORT migraphx_status migraphx_program_compile(migraphx_program_t program,
                                                           migraphx_target_t target,
                                                           migraphx_compile_options_t options);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_get_parameter_shapes(migraphx_program_parameter_shapes_t* out,
                                      migraphx_program_t program);
MIGRAPHX_C_EXPORT migraphx_status migraphx_program_get_output_shapes(migraphx_shapes_t* out,
                                                                     migraphx_program_t program);
MIGRAPHX_C_EXPORT migraphx_status migraphx_program_print(const_migraphx_program_t program);
MIGRAPHX_C_EXPORT migraphx_status migraphx_program_run(migraphx_arguments_t* out,
                                                       migraphx_program_t program,
                                                       migraphx_program_parameters_t params);
MIGRAPHX_C_EXPORT migraphx_status migraphx_program_equal(bool* out,
                                                         const_migraphx_program_t program,
                                                         const_migraphx_program_t x);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_program_experimental_get_context(migraphx_context_t* out, const_migraphx_program_t program);
MIGRAPHX_C_EXPORT migraphx_status migraphx_context_finish(const_migraphx_context_t context);

/* operation: `attributes` is a printf format of a JSON object whose keys may go unquoted,
 * e.g. "{axes: [%d], starts: [0]}"; NULL for none */
MIGRAPHX_C_EXPORT migraphx_status migraphx_operation_destroy(migraphx_operation_t operation);
MIGRAPHX_C_EXPORT migraphx_status migraphx_operation_assign_to(migraphx_operation_t output,
                                                               const_migraphx_operation_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_operation_create(migraphx_operation_t* operation,
                                                            const char* name,
                                                            const char* attributes,
                                                            ...);
MIGRAPHX_C_EXPORT migraphx_status migraphx_operation_name(char* out,
                                                          size_t out_size,
                                                          migraphx_operation_t operation);

/* programs on disk */
MIGRAPHX_C_EXPORT migraphx_status migraphx_load(migraphx_program_t* out,
                                                const char* name,
                                                migraphx_file_options_t options);
MIGRAPHX_C_EXPORT migraphx_status migraphx_save(migraphx_program_t p,
                                                const char* name,
                                                migraphx_file_options_t options);
MIGRAPHX_C_EXPORT migraphx_status migraphx_file_options_destroy(migraphx_file_options_t file_options);
MIGRAPHX_C_EXPORT migraphx_status migraphx_file_options_assign_to(migraphx_file_options_t output,
                                                                  const_migraphx_file_options_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_file_options_create(migraphx_file_options_t* file_options);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_file_options_set_file_format(migraphx_file_options_t file_options, const char* format);

/* compile options */
MIGRAPHX_C_EXPORT migraphx_status
migraphx_compile_options_destroy(migraphx_compile_options_t compile_options);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_compile_options_assign_to(migraphx_compile_options_t output,
                                   const_migraphx_compile_options_t input);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_compile_options_create(migraphx_compile_options_t* compile_options);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_compile_options_set_offload_copy(migraphx_compile_options_t compile_options, bool value);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_compile_options_set_fast_math(migraphx_compile_options_t compile_options, bool value);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_compile_options_set_exhaustive_tune_flag(migraphx_compile_options_t compile_options,
                                                  bool value);

/* ONNX */
MIGRAPHX_C_EXPORT migraphx_status migraphx_onnx_options_destroy(migraphx_onnx_options_t onnx_options);
MIGRAPHX_C_EXPORT migraphx_status migraphx_onnx_options_assign_to(migraphx_onnx_options_t output,
                                                                  const_migraphx_onnx_options_t input);
MIGRAPHX_C_EXPORT migraphx_status migraphx_onnx_options_create(migraphx_onnx_options_t* onnx_options);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_onnx_options_set_input_parameter_shape(migraphx_onnx_options_t onnx_options,
                                                const char* name,
                                                size_t* dims,
                                                size_t dims_size);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_onnx_options_set_default_dim_value(migraphx_onnx_options_t onnx_options, size_t value);
MIGRAPHX_C_EXPORT migraphx_status migraphx_parse_onnx(migraphx_program_t* out,
                                                      const char* name,
                                                      migraphx_onnx_options_t options);
MIGRAPHX_C_EXPORT migraphx_status migraphx_parse_onnx_buffer(migraphx_program_t* out,
                                                             const void* data,
                                                             size_t size,
                                                             migraphx_onnx_options_t options);

/* quantization; no operator names given means dot and convolution */
MIGRAPHX_C_EXPORT migraphx_status
migraphx_quantize_int8_options_destroy(migraphx_quantize_int8_options_t quantize_int8_options);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_quantize_int8_options_assign_to(migraphx_quantize_int8_options_t output,
                                         const_migraphx_quantize_int8_options_t input);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_quantize_int8_options_create(migraphx_quantize_int8_options_t* quantize_int8_options);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_quantize_int8_options_add_op_name(migraphx_quantize_int8_options_t quantize_int8_options,
                                           const char* name);
MIGRAPHX_C_EXPORT migraphx_status migraphx_quantize_int8_options_add_calibration_data(
    migraphx_quantize_int8_options_t quantize_int8_options, migraphx_program_parameters_t data);
MIGRAPHX_C_EXPORT migraphx_status migraphx_quantize_int8(migraphx_program_t prog,
                                                         migraphx_target_t target,
                                                         migraphx_quantize_int8_options_t options);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_quantize_fp8_options_destroy(migraphx_quantize_fp8_options_t quantize_fp8_options);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_quantize_fp8_options_assign_to(migraphx_quantize_fp8_options_t output,
                                        const_migraphx_quantize_fp8_options_t input);
MIGRAPHX_C_EXPORT migraphx_status
migraphx_quantize_fp8_options_create(migraphx_quantize_fp8_options_t* quantize_fp8_options);
MIGRAPHX_C_EXPORT migraphx_status migraphx_quantize_fp8_options_add_calibration_data(
    migraphx_quantize_fp8_options_t quantize_fp8_options, migraphx_program_parameters_t data);
MIGRAPHX_C_EXPORT migraphx_status migraphx_quantize_fp8(migraphx_program_t prog,
                                                        migraphx_target_t target,
                                                        migraphx_quantize_fp8_options_t options);
/* weight-only int4 (quantize_int4_weights of src/include/migraphx/quantization.hpp; the
 * reference's C header does not carry it yet) */
MIGRAPHX_C_EXPORT migraphx_status migraphx_quantize_int4_weights(migraphx_program_t prog);

#ifdef __cplusplus
}
#endif

#endif
