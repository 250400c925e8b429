// The C entry points declared in include/migraphx/migraphx.h.  Every handle is a struct holding
// the C++ object it stands for as its only member, so a pointer to an object that lives inside a
// container (a shape in a list, the main module of a program) can be handed out as a handle without
// a copy.  Exceptions stop at the boundary and become status codes (src/api/api.cpp:60-98).
#include <migraphx/migraphx.h>
#include <migraphx/json.hpp>
#include <migraphx/load_save.hpp>
#include <migraphx/onnx.hpp>
#include <migraphx/passes.hpp>
#include <migraphx/program.hpp>
#include <migraphx/register_target.hpp>
#include <algorithm>
#include <cctype>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <iostream>
#include <unordered_map>
#include <unordered_set>

namespace {

struct int8_options
{
    std::vector<migraphx::parameter_map> calibration;
    std::unordered_set<std::string> op_names;
};
struct fp8_options
{
    std::vector<migraphx::parameter_map> calibration;
};
// parameter shapes keep the program's parameter order
struct named_shapes
{
    std::vector<std::string> names;
    std::unordered_map<std::string, migraphx::shape> shapes;
};

} // namespace

#define MIGRAPHX_C_DEFINE_HANDLE(name, ...) \
    extern "C" struct migraphx_##name       \
    {                                       \
        __VA_ARGS__ object;                 \
    }

MIGRAPHX_C_DEFINE_HANDLE(shape, migraphx::shape);
MIGRAPHX_C_DEFINE_HANDLE(argument, migraphx::argument);
MIGRAPHX_C_DEFINE_HANDLE(target, migraphx::target);
MIGRAPHX_C_DEFINE_HANDLE(program_parameter_shapes, named_shapes);
MIGRAPHX_C_DEFINE_HANDLE(program_parameters, migraphx::parameter_map);
MIGRAPHX_C_DEFINE_HANDLE(arguments, std::vector<migraphx::argument>);
MIGRAPHX_C_DEFINE_HANDLE(shapes, std::vector<migraphx::shape>);
MIGRAPHX_C_DEFINE_HANDLE(instruction, migraphx::instruction_ref);
MIGRAPHX_C_DEFINE_HANDLE(instructions, std::vector<migraphx::instruction_ref>);
MIGRAPHX_C_DEFINE_HANDLE(module, migraphx::module);
MIGRAPHX_C_DEFINE_HANDLE(program, migraphx::program);
MIGRAPHX_C_DEFINE_HANDLE(operation, migraphx::operation);
MIGRAPHX_C_DEFINE_HANDLE(onnx_options, migraphx::onnx_options);
MIGRAPHX_C_DEFINE_HANDLE(file_options, migraphx::file_options);
MIGRAPHX_C_DEFINE_HANDLE(compile_options, migraphx::compile_options);
MIGRAPHX_C_DEFINE_HANDLE(quantize_int8_options, int8_options);
MIGRAPHX_C_DEFINE_HANDLE(quantize_fp8_options, fp8_options);
MIGRAPHX_C_DEFINE_HANDLE(context, migraphx::context);

namespace {

struct bad_param : std::runtime_error
{
    using std::runtime_error::runtime_error;
};
struct unknown_target : std::runtime_error
{
    using std::runtime_error::runtime_error;
};

template <class F>
migraphx_status guarded(const char* function, F f)
{
    auto report = [&](const char* what) { std::cerr << function << ": Error: " << what << std::endl; };
    try
    {
        f();
        return migraphx_status_success;
    }
    catch(const bad_param& e)
    {
        report(e.what());
        return migraphx_status_bad_param;
    }
    catch(const unknown_target& e)
    {
        report(e.what());
        return migraphx_status_unknown_target;
    }
    catch(const migraphx::exception& e)
    {
        report(e.what());
        return e.error > 0 ? static_cast<migraphx_status>(e.error) : migraphx_status_unknown_error;
    }
    catch(const std::exception& e)
    {
        report(e.what());
        return migraphx_status_unknown_error;
    }
    catch(...)
    {
        return migraphx_status_unknown_error;
    }
}

template <class T>
T& required(T* p, const char* name)
{
    if(p == nullptr)
        throw bad_param(std::string("Bad parameter ") + name + ": Null pointer");
    return *p;
}

// a handle whose object is `x` itself (no copy): the handle struct has `object` as its only member
template <class Handle, class T>
Handle* view_as(T* x)
{
    static_assert(sizeof(Handle) == sizeof(T), "a handle holds exactly its object");
    return reinterpret_cast<Handle*>(x);
}
template <class Handle, class T>
const Handle* view_as(const T* x)
{
    static_assert(sizeof(Handle) == sizeof(T), "a handle holds exactly its object");
    return reinterpret_cast<const Handle*>(x);
}

template <class Handle, class T>
Handle* make(T x)
{
    return new Handle{std::move(x)};
}

migraphx::shape::type_t element_type(migraphx_shape_datatype_t t)
{
    if(t == migraphx_shape_tuple_type)
        return migraphx::shape::tuple_type;
    if(t == migraphx_shape_fp4x2_type)
        return migraphx::shape::fp4x2_type;
    if(t >= migraphx_shape_bool_type and t <= migraphx_shape_fp8e5m2fnuz_type)
        return static_cast<migraphx::shape::type_t>(static_cast<int>(t) - 2);
    throw bad_param("Unknown type");
}

migraphx_shape_datatype_t element_type(migraphx::shape::type_t t)
{
    if(t == migraphx::shape::tuple_type)
        return migraphx_shape_tuple_type;
    if(t == migraphx::shape::fp4x2_type)
        return migraphx_shape_fp4x2_type;
    return static_cast<migraphx_shape_datatype_t>(static_cast<int>(t) + 2);
}

// The attribute text of migraphx_operation_create is JSON whose keys (and bare words that are not
// JSON literals) may go unquoted: {axes: [1], mode: same}.  Quote them.
std::string quote_bare_words(const std::string& text)
{
    std::string out;
    for(std::size_t i = 0; i < text.size();)
    {
        const char c = text[i];
        if(c == '"')
        {
            auto j = i + 1;
            while(j < text.size() and text[j] != '"')
                j += text[j] == '\\' ? 2 : 1;
            out.append(text, i, std::min(j + 1, text.size()) - i);
            i = j + 1;
        }
        else if(std::isalpha(static_cast<unsigned char>(c)) != 0 or c == '_')
        {
            // letters, digits, '_', '.', and "::" between the parts of a qualified name
            auto j = i;
            while(j < text.size())
            {
                if(std::isalnum(static_cast<unsigned char>(text[j])) != 0 or text[j] == '_' or text[j] == '.')
                    j++;
                else if(text[j] == ':' and j + 1 < text.size() and text[j + 1] == ':')
                    j += 2;
                else
                    break;
            }
            const auto word = text.substr(i, j - i);
            if(word == "true" or word == "false" or word == "null")
                out += word;
            else
                out += '"' + word + '"';
            i = j;
        }
        else
        {
            out += c;
            i++;
        }
    }
    return out;
}

migraphx::operation make_operation(const char* name, const char* attributes, va_list args)
{
    migraphx::value v = migraphx::value::object();
    if(attributes != nullptr)
    {
        va_list measure;
        va_copy(measure, args);
        const int n = std::vsnprintf(nullptr, 0, attributes, measure);
        va_end(measure);
        if(n < 0)
            throw bad_param("Bad parameter attributes: not a format string");
        std::string text(static_cast<std::size_t>(n) + 1, '\0');
        std::vsnprintf(&text[0], text.size(), attributes, args);
        text.resize(static_cast<std::size_t>(n));
        auto first = text.find_first_not_of(" \t\n");
        if(first != std::string::npos)
        {
            if(text[first] != '{')
                text = "{" + text + "}";
            v = migraphx::from_json_string(quote_bare_words(text));
        }
    }
    return migraphx::make_op(name, v);
}

} // namespace

#define API(function, ...) return guarded(#function, [&] { __VA_ARGS__ })

// destroy / assign_to of an owning handle
#define MIGRAPHX_C_OBJECT_LIFETIME(name)                                                     \
    extern "C" migraphx_status migraphx_##name##_destroy(migraphx_##name##_t name)           \
    {                                                                                        \
        API(migraphx_##name##_destroy, delete name;);                                        \
    }                                                                                        \
    extern "C" migraphx_status migraphx_##name##_assign_to(migraphx_##name##_t output,       \
                                                           const_migraphx_##name##_t input)  \
    {                                                                                        \
        API(migraphx_##name##_assign_to,                                                     \
            required(output, "output").object = required(input, "input").object;);           \
    }

MIGRAPHX_C_OBJECT_LIFETIME(shape)
MIGRAPHX_C_OBJECT_LIFETIME(argument)
MIGRAPHX_C_OBJECT_LIFETIME(target)
MIGRAPHX_C_OBJECT_LIFETIME(program_parameter_shapes)
MIGRAPHX_C_OBJECT_LIFETIME(program_parameters)
MIGRAPHX_C_OBJECT_LIFETIME(arguments)
MIGRAPHX_C_OBJECT_LIFETIME(shapes)
MIGRAPHX_C_OBJECT_LIFETIME(instruction)
MIGRAPHX_C_OBJECT_LIFETIME(instructions)
MIGRAPHX_C_OBJECT_LIFETIME(program)
MIGRAPHX_C_OBJECT_LIFETIME(operation)
MIGRAPHX_C_OBJECT_LIFETIME(onnx_options)
MIGRAPHX_C_OBJECT_LIFETIME(file_options)
MIGRAPHX_C_OBJECT_LIFETIME(compile_options)
MIGRAPHX_C_OBJECT_LIFETIME(quantize_int8_options)
MIGRAPHX_C_OBJECT_LIFETIME(quantize_fp8_options)

// ----------------------------------------------------------------------- shape

extern "C" migraphx_status migraphx_shape_create(migraphx_shape_t* shape,
                                                 migraphx_shape_datatype_t type,
                                                 size_t* lengths,
                                                 size_t lengths_size)
{
    API(migraphx_shape_create, {
        if(lengths == nullptr and lengths_size != 0)
            throw bad_param("Bad parameter lengths: Null pointer");
        required(shape, "shape") = make<migraphx_shape>(migraphx::shape{
            element_type(type), std::vector<std::size_t>(lengths, lengths + lengths_size)});
    });
}

extern "C" migraphx_status migraphx_shape_create_with_strides(migraphx_shape_t* shape,
                                                              migraphx_shape_datatype_t type,
                                                              size_t* lengths,
                                                              size_t lengths_size,
                                                              size_t* strides,
                                                              size_t strides_size)
{
    API(migraphx_shape_create_with_strides, {
        if(lengths == nullptr and lengths_size != 0)
            throw bad_param("Bad parameter lengths: Null pointer");
        if(strides == nullptr and strides_size != 0)
            throw bad_param("Bad parameter strides: Null pointer");
        required(shape, "shape") = make<migraphx_shape>(
            migraphx::shape{element_type(type),
                            std::vector<std::size_t>(lengths, lengths + lengths_size),
                            std::vector<std::size_t>(strides, strides + strides_size)});
    });
}

extern "C" migraphx_status migraphx_shape_create_scalar(migraphx_shape_t* shape,
                                                        migraphx_shape_datatype_t type)
{
    API(migraphx_shape_create_scalar,
        required(shape, "shape") = make<migraphx_shape>(migraphx::shape{element_type(type)}););
}

extern "C" migraphx_status
migraphx_shape_lengths(const size_t** out, size_t* out_size, const_migraphx_shape_t shape)
{
    API(migraphx_shape_lengths, {
        const auto& lens           = required(shape, "shape").object.lens();
        required(out, "out")       = lens.data();
        required(out_size, "out_size") = lens.size();
    });
}

extern "C" migraphx_status
migraphx_shape_strides(const size_t** out, size_t* out_size, const_migraphx_shape_t shape)
{
    API(migraphx_shape_strides, {
        const auto& strides        = required(shape, "shape").object.strides();
        required(out, "out")       = strides.data();
        required(out_size, "out_size") = strides.size();
    });
}

extern "C" migraphx_status migraphx_shape_type(migraphx_shape_datatype_t* out,
                                               const_migraphx_shape_t shape)
{
    API(migraphx_shape_type,
        required(out, "out") = element_type(required(shape, "shape").object.type()););
}

extern "C" migraphx_status migraphx_shape_elements(size_t* out, const_migraphx_shape_t shape)
{
    API(migraphx_shape_elements, required(out, "out") = required(shape, "shape").object.elements(););
}

extern "C" migraphx_status migraphx_shape_bytes(size_t* out, const_migraphx_shape_t shape)
{
    API(migraphx_shape_bytes, required(out, "out") = required(shape, "shape").object.bytes(););
}

extern "C" migraphx_status migraphx_shape_ndim(size_t* out, const_migraphx_shape_t shape)
{
    API(migraphx_shape_ndim, required(out, "out") = required(shape, "shape").object.ndim(););
}

extern "C" migraphx_status
migraphx_shape_equal(bool* out, const_migraphx_shape_t shape, const_migraphx_shape_t x)
{
    API(migraphx_shape_equal,
        required(out, "out") = required(shape, "shape").object == required(x, "x").object;);
}

extern "C" migraphx_status migraphx_shape_standard(bool* out, const_migraphx_shape_t shape)
{
    API(migraphx_shape_standard, required(out, "out") = required(shape, "shape").object.standard(););
}

extern "C" migraphx_status migraphx_shape_dynamic(bool* out, const_migraphx_shape_t shape)
{
    API(migraphx_shape_dynamic, {
        required(shape, "shape");
        required(out, "out") = false;
    });
}

extern "C" migraphx_status migraphx_shape_index(size_t* out, const_migraphx_shape_t shape, size_t i)
{
    API(migraphx_shape_index, required(out, "out") = required(shape, "shape").object.index(i););
}

// -------------------------------------------------------------------- argument

extern "C" migraphx_status migraphx_argument_create(migraphx_argument_t* argument,
                                                    const_migraphx_shape_t shape,
                                                    void* buffer)
{
    API(migraphx_argument_create,
        required(argument, "argument") = make<migraphx_argument>(
            migraphx::argument{required(shape, "shape").object, buffer}););
}

extern "C" migraphx_status migraphx_argument_create_empty(migraphx_argument_t* argument,
                                                          const_migraphx_shape_t shape)
{
    API(migraphx_argument_create_empty,
        required(argument, "argument") =
            make<migraphx_argument>(migraphx::argument{required(shape, "shape").object}););
}

extern "C" migraphx_status migraphx_argument_shape(const_migraphx_shape_t* out,
                                                   const_migraphx_argument_t argument)
{
    API(migraphx_argument_shape,
        required(out, "out") =
            view_as<migraphx_shape>(&required(argument, "argument").object.get_shape()););
}

extern "C" migraphx_status migraphx_argument_buffer(char** out, const_migraphx_argument_t argument)
{
    API(migraphx_argument_buffer,
        required(out, "out") = required(argument, "argument").object.data(););
}

extern "C" migraphx_status
migraphx_argument_equal(bool* out, const_migraphx_argument_t argument, const_migraphx_argument_t x)
{
    API(migraphx_argument_equal, {
        const auto& a = required(argument, "argument").object;
        const auto& b = required(x, "x").object;
        bool same     = a.get_shape() == b.get_shape() and a.empty() == b.empty();
        if(same and not a.empty())
            same = std::memcmp(a.data(), b.data(), a.get_shape().bytes()) == 0;
        required(out, "out") = same;
    });
}

extern "C" migraphx_status migraphx_argument_save(const_migraphx_argument_t a, const char* filename)
{
    API(migraphx_argument_save,
        migraphx::save_argument(required(a, "a").object, &required(filename, "filename")););
}

extern "C" migraphx_status migraphx_argument_load(migraphx_argument_t* out, const char* filename)
{
    API(migraphx_argument_load,
        required(out, "out") =
            make<migraphx_argument>(migraphx::load_argument(&required(filename, "filename"))););
}

extern "C" migraphx_status
migraphx_argument_generate(migraphx_argument_t* out, const_migraphx_shape_t s, size_t seed)
{
    API(migraphx_argument_generate,
        required(out, "out") =
            make<migraphx_argument>(migraphx::generate_argument(required(s, "s").object, seed)););
}

// ---------------------------------------------------------------------- target

extern "C" migraphx_status migraphx_target_create(migraphx_target_t* target, const char* name)
{
    API(migraphx_target_create, {
        const std::string n = &required(name, "name");
        // the reference's name for the device target selects this build's
        const std::string resolved = n == "gpu" ? "mi355" : n;
        migraphx::target t;
        try
        {
            t = migraphx::make_target(resolved);
        }
        catch(const migraphx::exception& e)
        {
            throw unknown_target(e.what());
        }
        required(target, "target") = make<migraphx_target>(std::move(t));
    });
}

// ----------------------------------------------------- parameter shapes / values

extern "C" migraphx_status
migraphx_program_parameter_shapes_size(size_t* out,
                                       migraphx_program_parameter_shapes_t program_parameter_shapes)
{
    API(migraphx_program_parameter_shapes_size,
        required(out, "out") =
            required(program_parameter_shapes, "program_parameter_shapes").object.names.size(););
}

extern "C" migraphx_status
migraphx_program_parameter_shapes_get(const_migraphx_shape_t* out,
                                      migraphx_program_parameter_shapes_t program_parameter_shapes,
                                      const char* name)
{
    API(migraphx_program_parameter_shapes_get, {
        auto& shapes = required(program_parameter_shapes, "program_parameter_shapes").object.shapes;
        auto it      = shapes.find(&required(name, "name"));
        if(it == shapes.end())
            throw bad_param(std::string("Bad parameter name: no parameter '") + name + "'");
        required(out, "out") = view_as<migraphx_shape>(&it->second);
    });
}

extern "C" migraphx_status
migraphx_program_parameter_shapes_names(const char** out,
                                        migraphx_program_parameter_shapes_t program_parameter_shapes)
{
    API(migraphx_program_parameter_shapes_names, {
        auto& names = required(program_parameter_shapes, "program_parameter_shapes").object.names;
        required(out, "out");
        for(std::size_t i = 0; i < names.size(); i++)
            out[i] = names[i].c_str();
    });
}

extern "C" migraphx_status
migraphx_program_parameters_create(migraphx_program_parameters_t* program_parameters)
{
    API(migraphx_program_parameters_create,
        required(program_parameters, "program_parameters") =
            make<migraphx_program_parameters>(migraphx::parameter_map{}););
}

extern "C" migraphx_status
migraphx_program_parameters_add(migraphx_program_parameters_t program_parameters,
                                const char* name,
                                const_migraphx_argument_t argument)
{
    API(migraphx_program_parameters_add,
        required(program_parameters, "program_parameters").object[&required(name, "name")] =
            required(argument, "argument").object;);
}

// ----------------------------------------------------------------------- lists

extern "C" migraphx_status migraphx_arguments_size(size_t* out, migraphx_arguments_t arguments)
{
    API(migraphx_arguments_size,
        required(out, "out") = required(arguments, "arguments").object.size(););
}

extern "C" migraphx_status
migraphx_arguments_get(const_migraphx_argument_t* out, migraphx_arguments_t arguments, size_t idx)
{
    API(migraphx_arguments_get, {
        auto& list = required(arguments, "arguments").object;
        if(idx >= list.size())
            throw bad_param("Bad parameter idx: out of range");
        required(out, "out") = view_as<migraphx_argument>(&list[idx]);
    });
}

extern "C" migraphx_status migraphx_shapes_size(size_t* out, migraphx_shapes_t shapes)
{
    API(migraphx_shapes_size, required(out, "out") = required(shapes, "shapes").object.size(););
}

extern "C" migraphx_status
migraphx_shapes_get(const_migraphx_shape_t* out, migraphx_shapes_t shapes, size_t idx)
{
    API(migraphx_shapes_get, {
        auto& list = required(shapes, "shapes").object;
        if(idx >= list.size())
            throw bad_param("Bad parameter idx: out of range");
        required(out, "out") = view_as<migraphx_shape>(&list[idx]);
    });
}

extern "C" migraphx_status migraphx_instructions_create(migraphx_instructions_t* instructions,
                                                        const const_migraphx_instruction_t* ptr,
                                                        size_t size)
{
    API(migraphx_instructions_create, {
        if(ptr == nullptr and size != 0)
            throw bad_param("Bad parameter ptr: Null pointer");
        std::vector<migraphx::instruction_ref> list;
        for(std::size_t i = 0; i < size; i++)
            list.push_back(required(ptr[i], "ptr").object);
        required(instructions, "instructions") = make<migraphx_instructions>(std::move(list));
    });
}

// ---------------------------------------------------------------------- module

extern "C" migraphx_status migraphx_module_print(const_migraphx_module_t module)
{
    API(migraphx_module_print, std::cout << required(module, "module").object << std::endl;);
}

extern "C" migraphx_status migraphx_module_add_instruction(migraphx_instruction_t* out,
                                                           migraphx_module_t module,
                                                           migraphx_operation_t op,
                                                           migraphx_instructions_t args)
{
    API(migraphx_module_add_instruction,
        required(out, "out") = make<migraphx_instruction>(required(module, "module").object.add_instruction(
            required(op, "op").object, required(args, "args").object)););
}

extern "C" migraphx_status migraphx_module_add_literal(migraphx_instruction_t* out,
                                                       migraphx_module_t module,
                                                       const_migraphx_shape_t shape,
                                                       const char* buffer)
{
    API(migraphx_module_add_literal,
        required(out, "out") = make<migraphx_instruction>(required(module, "module").object.add_literal(
            migraphx::literal{required(shape, "shape").object, &required(buffer, "buffer")})););
}

extern "C" migraphx_status migraphx_module_add_parameter(migraphx_instruction_t* out,
                                                         migraphx_module_t module,
                                                         const char* name,
                                                         const_migraphx_shape_t shape)
{
    API(migraphx_module_add_parameter,
        required(out, "out") = make<migraphx_instruction>(required(module, "module").object.add_parameter(
            &required(name, "name"), required(shape, "shape").object)););
}

extern "C" migraphx_status migraphx_module_add_return(migraphx_instruction_t* out,
                                                      migraphx_module_t module,
                                                      migraphx_instructions_t args)
{
    API(migraphx_module_add_return,
        required(out, "out") = make<migraphx_instruction>(
            required(module, "module").object.add_return(required(args, "args").object)););
}

// --------------------------------------------------------------------- program

extern "C" migraphx_status migraphx_program_create(migraphx_program_t* program)
{
    API(migraphx_program_create,
        required(program, "program") = make<migraphx_program>(migraphx::program{}););
}

extern "C" migraphx_status migraphx_program_get_main_module(migraphx_module_t* out,
                                                            migraphx_program_t program)
{
    API(migraphx_program_get_main_module,
        required(out, "out") =
            view_as<migraphx_module>(required(program, "program").object.get_main_module()););
}

extern "C" migraphx_status migraphx_program_compile(migraphx_program_t program,
                                                    migraphx_target_t target,
                                                    migraphx_compile_options_t options)
{
    API(migraphx_program_compile,
        required(program, "program")
            .object.compile(required(target, "target").object,
                            options == nullptr ? migraphx::compile_options{} : options->object););
}

extern "C" migraphx_status
migraphx_program_get_parameter_shapes(migraphx_program_parameter_shapes_t* out,
                                      migraphx_program_t program)
{
    API(migraphx_program_get_parameter_shapes, {
        auto& p = required(program, "program").object;
        named_shapes r;
        r.names  = p.get_parameter_names();
        r.shapes = p.get_parameter_shapes();
        required(out, "out") = make<migraphx_program_parameter_shapes>(std::move(r));
    });
}

extern "C" migraphx_status migraphx_program_get_output_shapes(migraphx_shapes_t* out,
                                                              migraphx_program_t program)
{
    API(migraphx_program_get_output_shapes,
        required(out, "out") =
            make<migraphx_shapes>(required(program, "program").object.get_output_shapes()););
}

extern "C" migraphx_status migraphx_program_print(const_migraphx_program_t program)
{
    API(migraphx_program_print, std::cout << required(program, "program").object << std::endl;);
}

extern "C" migraphx_status migraphx_program_run(migraphx_arguments_t* out,
                                                migraphx_program_t program,
                                                migraphx_program_parameters_t params)
{
    API(migraphx_program_run, {
        auto& p      = required(program, "program").object;
        auto results = p.eval(required(params, "params").object);
        p.finish();
        required(out, "out") = make<migraphx_arguments>(std::move(results));
    });
}

extern "C" migraphx_status
migraphx_program_equal(bool* out, const_migraphx_program_t program, const_migraphx_program_t x)
{
    API(migraphx_program_equal,
        required(out, "out") = required(program, "program").object == required(x, "x").object;);
}

extern "C" migraphx_status
migraphx_program_experimental_get_context(migraphx_context_t* out, const_migraphx_program_t program)
{
    // the context is shared with the program: the handle refers into it
    API(migraphx_program_experimental_get_context,
        required(out, "out") = view_as<migraphx_context>(
            &const_cast<migraphx::program&>(required(program, "program").object).get_context()););
}

extern "C" migraphx_status migraphx_context_finish(const_migraphx_context_t context)
{
    API(migraphx_context_finish, required(context, "context").object.finish(););
}

// ------------------------------------------------------------------- operation

extern "C" migraphx_status migraphx_operation_create(migraphx_operation_t* operation,
                                                     const char* name,
                                                     const char* attributes,
                                                     ...)
{
    va_list args;
    va_start(args, attributes);
    auto status = guarded("migraphx_operation_create", [&] {
        required(operation, "operation") =
            make<migraphx_operation>(make_operation(&required(name, "name"), attributes, args));
    });
    va_end(args);
    return status;
}

extern "C" migraphx_status
migraphx_operation_name(char* out, size_t out_size, migraphx_operation_t operation)
{
    API(migraphx_operation_name, {
        required(out, "out");
        if(out_size == 0)
            throw bad_param("Bad parameter out_size: no room for the name");
        const auto name = required(operation, "operation").object.name();
        const auto n    = std::min(name.size(), out_size - 1);
        std::memcpy(out, name.data(), n);
        out[n] = '\0';
    });
}

// ------------------------------------------------------------ programs on disk

extern "C" migraphx_status
migraphx_load(migraphx_program_t* out, const char* name, migraphx_file_options_t options)
{
    API(migraphx_load,
        required(out, "out") = make<migraphx_program>(migraphx::load(
            &required(name, "name"), options == nullptr ? migraphx::file_options{} : options->object)););
}

extern "C" migraphx_status
migraphx_save(migraphx_program_t p, const char* name, migraphx_file_options_t options)
{
    API(migraphx_save,
        migraphx::save(required(p, "p").object,
                       &required(name, "name"),
                       options == nullptr ? migraphx::file_options{} : options->object););
}

extern "C" migraphx_status migraphx_file_options_create(migraphx_file_options_t* file_options)
{
    API(migraphx_file_options_create,
        required(file_options, "file_options") = make<migraphx_file_options>(migraphx::file_options{}););
}

extern "C" migraphx_status
migraphx_file_options_set_file_format(migraphx_file_options_t file_options, const char* format)
{
    API(migraphx_file_options_set_file_format,
        required(file_options, "file_options").object.format = &required(format, "format"););
}

// ------------------------------------------------------------- compile options

extern "C" migraphx_status migraphx_compile_options_create(migraphx_compile_options_t* compile_options)
{
    API(migraphx_compile_options_create,
        required(compile_options, "compile_options") =
            make<migraphx_compile_options>(migraphx::compile_options{}););
}

extern "C" migraphx_status
migraphx_compile_options_set_offload_copy(migraphx_compile_options_t compile_options, bool value)
{
    API(migraphx_compile_options_set_offload_copy,
        required(compile_options, "compile_options").object.offload_copy = value;);
}

extern "C" migraphx_status
migraphx_compile_options_set_fast_math(migraphx_compile_options_t compile_options, bool value)
{
    API(migraphx_compile_options_set_fast_math,
        required(compile_options, "compile_options").object.fast_math = value;);
}

extern "C" migraphx_status
migraphx_compile_options_set_exhaustive_tune_flag(migraphx_compile_options_t compile_options, bool value)
{
    API(migraphx_compile_options_set_exhaustive_tune_flag,
        required(compile_options, "compile_options").object.exhaustive_tune = value;);
}

// ------------------------------------------------------------------------ ONNX

extern "C" migraphx_status migraphx_onnx_options_create(migraphx_onnx_options_t* onnx_options)
{
    API(migraphx_onnx_options_create,
        required(onnx_options, "onnx_options") = make<migraphx_onnx_options>(migraphx::onnx_options{}););
}

extern "C" migraphx_status
migraphx_onnx_options_set_input_parameter_shape(migraphx_onnx_options_t onnx_options,
                                                const char* name,
                                                size_t* dims,
                                                size_t dims_size)
{
    API(migraphx_onnx_options_set_input_parameter_shape, {
        if(dims == nullptr and dims_size != 0)
            throw bad_param("Bad parameter dims: Null pointer");
        required(onnx_options, "onnx_options").object.map_input_dims[&required(name, "name")] =
            std::vector<std::size_t>(dims, dims + dims_size);
    });
}

extern "C" migraphx_status
migraphx_onnx_options_set_default_dim_value(migraphx_onnx_options_t onnx_options, size_t value)
{
    API(migraphx_onnx_options_set_default_dim_value,
        required(onnx_options, "onnx_options").object.default_dim_value = value;);
}

extern "C" migraphx_status
migraphx_parse_onnx(migraphx_program_t* out, const char* name, migraphx_onnx_options_t options)
{
    API(migraphx_parse_onnx,
        required(out, "out") = make<migraphx_program>(migraphx::parse_onnx(
            &required(name, "name"), options == nullptr ? migraphx::onnx_options{} : options->object)););
}

extern "C" migraphx_status migraphx_parse_onnx_buffer(migraphx_program_t* out,
                                                      const void* data,
                                                      size_t size,
                                                      migraphx_onnx_options_t options)
{
    API(migraphx_parse_onnx_buffer,
        required(out, "out") = make<migraphx_program>(migraphx::parse_onnx_buffer(
            &required(static_cast<const char*>(data), "data"),
            size,
            options == nullptr ? migraphx::onnx_options{} : options->object)););
}

// ---------------------------------------------------------------- quantization

extern "C" migraphx_status
migraphx_quantize_int8_options_create(migraphx_quantize_int8_options_t* quantize_int8_options)
{
    API(migraphx_quantize_int8_options_create,
        required(quantize_int8_options, "quantize_int8_options") =
            make<migraphx_quantize_int8_options>(int8_options{}););
}

extern "C" migraphx_status
migraphx_quantize_int8_options_add_op_name(migraphx_quantize_int8_options_t quantize_int8_options,
                                           const char* name)
{
    API(migraphx_quantize_int8_options_add_op_name,
        required(quantize_int8_options, "quantize_int8_options")
            .object.op_names.insert(&required(name, "name")););
}

extern "C" migraphx_status migraphx_quantize_int8_options_add_calibration_data(
    migraphx_quantize_int8_options_t quantize_int8_options, migraphx_program_parameters_t data)
{
    API(migraphx_quantize_int8_options_add_calibration_data,
        required(quantize_int8_options, "quantize_int8_options")
            .object.calibration.push_back(required(data, "data").object););
}

extern "C" migraphx_status migraphx_quantize_int8(migraphx_program_t prog,
                                                  migraphx_target_t target,
                                                  migraphx_quantize_int8_options_t options)
{
    API(migraphx_quantize_int8, {
        auto& o = required(options, "options").object;
        if(o.op_names.empty())
            o.op_names = {"dot", "convolution"};
        migraphx::quantize_int8(
            required(prog, "prog").object, required(target, "target").object, o.calibration, o.op_names);
    });
}

extern "C" migraphx_status
migraphx_quantize_fp8_options_create(migraphx_quantize_fp8_options_t* quantize_fp8_options)
{
    API(migraphx_quantize_fp8_options_create,
        required(quantize_fp8_options, "quantize_fp8_options") =
            make<migraphx_quantize_fp8_options>(fp8_options{}););
}

extern "C" migraphx_status migraphx_quantize_fp8_options_add_calibration_data(
    migraphx_quantize_fp8_options_t quantize_fp8_options, migraphx_program_parameters_t data)
{
    API(migraphx_quantize_fp8_options_add_calibration_data,
        required(quantize_fp8_options, "quantize_fp8_options")
            .object.calibration.push_back(required(data, "data").object););
}

extern "C" migraphx_status migraphx_quantize_fp8(migraphx_program_t prog,
                                                 migraphx_target_t target,
                                                 migraphx_quantize_fp8_options_t options)
{
    API(migraphx_quantize_fp8,
        migraphx::quantize_fp8(required(prog, "prog").object,
                               required(target, "target").object,
                               required(options, "options").object.calibration););
}

extern "C" migraphx_status migraphx_quantize_int4_weights(migraphx_program_t prog)
{
    API(migraphx_quantize_int4_weights, migraphx::quantize_int4_weights(required(prog, "prog").object););
}
