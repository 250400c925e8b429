// Python surface of the host layer: the part of the reference's `migraphx` module
// (src/py/migraphx_py.cpp:362-626, :795-844) that builds, quantizes, compiles and runs a program
// on the quantized-GEMM path.  Same class and function names, argument names and defaults, so a
// script written against the reference runs against this module; get_target("gpu") names the
// MI355X target here.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>
#include <migraphx/make_op.hpp>
#include <migraphx/mi355/target.hpp>
#include <migraphx/load_save.hpp>
#include <migraphx/onnx.hpp>
#include <migraphx/ops.hpp>
#include <migraphx/passes.hpp>
#include <migraphx/program.hpp>
#include <migraphx/register_target.hpp>
#include <cstring>
#include <iostream>
#include <sstream>

namespace py = pybind11;
using migraphx::argument;
using migraphx::instruction_ref;
using migraphx::shape;
using migraphx::value;

namespace {

template <class T>
std::string to_string(const T& x)
{
    std::stringstream ss;
    ss << x;
    return ss.str();
}

// Python objects of make_op's keyword arguments (to_value of src/py/migraphx_py.cpp:101-180)
value to_value(const py::handle& h)
{
    if(py::isinstance<py::bool_>(h))
        return value(h.cast<bool>());
    if(py::isinstance<py::int_>(h))
        return value(h.cast<int64_t>());
    if(py::isinstance<py::float_>(h))
        return value(h.cast<double>());
    if(py::isinstance<py::str>(h))
        return value(h.cast<std::string>());
    if(py::isinstance<shape::type_t>(h))
        return value(h.cast<shape::type_t>());
    if(py::isinstance<py::dict>(h))
    {
        value v = value::object();
        for(auto item : h.cast<py::dict>())
            v.push_back(value(item.first.cast<std::string>(), to_value(item.second)));
        return v;
    }
    if(py::isinstance<py::list>(h) or py::isinstance<py::tuple>(h))
    {
        value v = value::array();
        for(auto item : h)
            v.push_back(to_value(item));
        return v;
    }
    throw py::type_error("migraphx: cannot convert " + py::repr(h).cast<std::string>() + " to an attribute");
}

py::object to_py_object(const value& v)
{
    switch(v.kind())
    {
    case value::null_kind: return py::none();
    case value::bool_kind: return py::bool_(v.to<bool>());
    case value::int_kind: return py::int_(v.to<int64_t>());
    case value::float_kind: return py::float_(v.to<double>());
    case value::string_kind: return py::str(v.to<std::string>());
    case value::array_kind: {
        py::list l;
        for(const auto& x : v.items())
            l.append(to_py_object(x));
        return std::move(l);
    }
    default: {
        py::dict d;
        for(const auto& x : v.items())
            d[py::str(x.get_key())] = to_py_object(x);
        return std::move(d);
    }
    }
}

// numpy's format characters (buffer protocol) for the element types that have one
std::string format_of(shape::type_t t)
{
    switch(t)
    {
    case shape::bool_type: return "?";
    case shape::half_type: return "e";
    case shape::float_type: return "f";
    case shape::double_type: return "d";
    case shape::uint8_type: return "B";
    case shape::int8_type: return "b";
    case shape::uint16_type: return "H";
    case shape::int16_type: return "h";
    case shape::int32_type: return "i";
    case shape::uint32_type: return "I";
    case shape::int64_type: return "q";
    case shape::uint64_type: return "Q";
    default: MIGRAPHX_THROW("migraphx: " + shape::type_name(t) + " tensors have no numpy element type");
    }
}

shape::type_t type_of(const std::string& format, std::size_t itemsize)
{
    const char c = format.empty() ? ' ' : format.back();
    switch(c)
    {
    case '?': return shape::bool_type;
    case 'e': return shape::half_type;
    case 'f': return shape::float_type;
    case 'd': return shape::double_type;
    case 'B': return shape::uint8_type;
    case 'b': return shape::int8_type;
    case 'H': return shape::uint16_type;
    case 'h': return shape::int16_type;
    case 'i': return shape::int32_type;
    case 'I': return shape::uint32_type;
    case 'l': return itemsize == 4 ? shape::int32_type : shape::int64_type;
    case 'L': return itemsize == 4 ? shape::uint32_type : shape::uint64_type;
    case 'q': return shape::int64_type;
    case 'Q': return shape::uint64_type;
    default: MIGRAPHX_THROW("migraphx: unsupported buffer element format '" + format + "'");
    }
}

shape to_shape(const py::buffer_info& info)
{
    const auto t = type_of(info.format, static_cast<std::size_t>(info.itemsize));
    std::vector<std::size_t> lens(info.shape.begin(), info.shape.end());
    std::vector<std::size_t> strides;
    for(auto s : info.strides)
    {
        if(s < 0 or s % info.itemsize != 0)
            MIGRAPHX_THROW("migraphx: buffers with negative or unaligned strides are not supported");
        strides.push_back(static_cast<std::size_t>(s / info.itemsize));
    }
    if(lens.empty())
        return shape{t};
    return shape{t, lens, strides};
}

py::buffer_info to_buffer_info(argument& a)
{
    const shape& s = a.get_shape();
    std::vector<py::ssize_t> lens(s.lens().begin(), s.lens().end());
    std::vector<py::ssize_t> strides;
    for(auto x : s.strides())
        strides.push_back(static_cast<py::ssize_t>(x * s.type_size()));
    return py::buffer_info(a.data(), static_cast<py::ssize_t>(s.type_size()), format_of(s.type()),
                           static_cast<py::ssize_t>(s.ndim()), lens, strides);
}

migraphx::parameter_map to_parameter_map(const py::dict& params)
{
    migraphx::parameter_map pm;
    for(auto x : params)
    {
        auto key = x.first.cast<std::string>();
        if(py::isinstance<argument>(x.second))
        {
            pm[key] = x.second.cast<argument>();
            continue;
        }
        py::buffer b         = x.second.cast<py::buffer>();
        py::buffer_info info = b.request();
        pm[key]              = argument(to_shape(info), info.ptr);
    }
    return pm;
}

// equal shapes and equal element values (host tensors)
bool same(const argument& a, const argument& b)
{
    if(a.get_shape().type() != b.get_shape().type() or a.get_shape().lens() != b.get_shape().lens())
        return false;
    return a.to_vector<double>() == b.to_vector<double>();
}

migraphx::target get_target(const std::string& name)
{
    return migraphx::make_target(name == "gpu" ? "mi355" : name);
}

} // namespace

PYBIND11_MODULE(migraphx, m)
{
    py::register_exception<migraphx::exception>(m, "MigraphxError", PyExc_RuntimeError);

    py::class_<shape> shape_cls(m, "shape");
    py::enum_<shape::type_t>(shape_cls, "type_t")
        .value("bool_type", shape::bool_type)
        .value("half_type", shape::half_type)
        .value("float_type", shape::float_type)
        .value("double_type", shape::double_type)
        .value("uint8_type", shape::uint8_type)
        .value("int8_type", shape::int8_type)
        .value("uint16_type", shape::uint16_type)
        .value("int16_type", shape::int16_type)
        .value("int32_type", shape::int32_type)
        .value("int64_type", shape::int64_type)
        .value("uint32_type", shape::uint32_type)
        .value("uint64_type", shape::uint64_type)
        .value("fp8e4m3fn_type", shape::fp8e4m3fn_type)
        .value("fp8e5m2_type", shape::fp8e5m2_type)
        .value("bf16_type", shape::bf16_type)
        .value("fp4x2_type", shape::fp4x2_type);
    shape_cls
        .def(py::init([](const py::kwargs& kwargs) {
            std::string type = "float";
            std::vector<std::size_t> lens{1};
            if(kwargs.contains("type"))
                type = kwargs["type"].cast<std::string>();
            if(kwargs.contains("lens"))
                lens = kwargs["lens"].cast<std::vector<std::size_t>>();
            const auto t = shape::parse_type(type);
            if(kwargs.contains("strides"))
                return shape(t, lens, kwargs["strides"].cast<std::vector<std::size_t>>());
            if(kwargs.contains("permutation"))
                return shape::from_permutation(t, lens, kwargs["permutation"].cast<std::vector<int64_t>>());
            return shape(t, lens);
        }))
        .def("type", &shape::type)
        .def("lens", &shape::lens)
        .def("strides", &shape::strides)
        .def("ndim", &shape::ndim)
        .def("elements", &shape::elements)
        .def("bytes", &shape::bytes)
        .def("type_string", &shape::type_string)
        .def("type_size", [](const shape& x) { return x.type_size(); })
        .def("packed", &shape::packed)
        .def("transposed", &shape::transposed)
        .def("broadcasted", &shape::broadcasted)
        .def("standard", &shape::standard)
        .def("scalar", &shape::scalar)
        .def("__eq__", [](const shape& a, const shape& b) { return a == b; })
        .def("__ne__", [](const shape& a, const shape& b) { return a != b; })
        .def("__repr__", [](const shape& s) { return to_string(s); });

    py::class_<argument>(m, "argument", py::buffer_protocol())
        .def_buffer([](argument& x) -> py::buffer_info { return to_buffer_info(x); })
        // the argument keeps its own copy, so the Python object it came from may go away
        .def(py::init([](const py::buffer& b) {
            py::buffer_info info = b.request();
            const shape s        = to_shape(info);
            argument view(s, info.ptr);
            return migraphx::op::contiguous{}.compute(shape{s.type(), s.lens()}, {view});
        }))
        .def("get_shape", &argument::get_shape)
        .def("data_ptr", [](argument& x) { return reinterpret_cast<std::uintptr_t>(x.data()); })
        .def("tolist", [](argument& x) { return x.to_vector<double>(); })
        .def("__eq__", [](const argument& a, const argument& b) { return same(a, b); })
        .def("__ne__", [](const argument& a, const argument& b) { return not same(a, b); })
        .def("__repr__", [](const argument& x) { return to_string(x); });

    py::class_<migraphx::target>(m, "target").def("name", &migraphx::target::name);

    py::class_<migraphx::operation>(m, "op")
        .def(py::init([](const std::string& name, const py::kwargs& kwargs) {
            value v = value::object();
            for(auto item : kwargs)
                v.push_back(value(item.first.cast<std::string>(), to_value(item.second)));
            return migraphx::make_op(name, v);
        }))
        .def("name", &migraphx::operation::name)
        .def("values", [](const migraphx::operation& o) { return to_py_object(o.to_value()); })
        .def("__repr__", [](const migraphx::operation& o) { return to_string(o); });

    py::class_<instruction_ref>(m, "instruction_ref")
        .def("shape", [](instruction_ref i) { return i->get_shape(); })
        .def("op", [](instruction_ref i) { return i->get_operator(); })
        .def("inputs", [](instruction_ref i) { return i->inputs(); })
        .def("outputs", [](instruction_ref i) { return i->outputs(); })
        .def("name", [](instruction_ref i) { return i->name(); })
        .def("__eq__", [](instruction_ref a, instruction_ref b) { return a == b; });

    py::class_<migraphx::module, std::unique_ptr<migraphx::module, py::nodelete>>(m, "module")
        .def("print", [](const migraphx::module& mm) { std::cout << mm << std::endl; })
        .def(
            "add_instruction",
            [](migraphx::module& mm, const migraphx::operation& op, std::vector<instruction_ref>& args) {
                return mm.add_instruction(op, args);
            },
            py::arg("op"),
            py::arg("args"))
        .def(
            "add_literal",
            [](migraphx::module& mm, const argument& a) {
                argument dense = migraphx::op::contiguous{}.compute(
                    shape{a.get_shape().type(), a.get_shape().lens()}, {a});
                return mm.add_literal(migraphx::literal{dense.get_shape(), dense.data()});
            },
            py::arg("data"))
        .def(
            "add_literal",
            [](migraphx::module& mm, const py::buffer& data) {
                py::buffer_info info = data.request();
                const shape s        = to_shape(info);
                argument dense       = migraphx::op::contiguous{}.compute(shape{s.type(), s.lens()},
                                                                    {argument(s, info.ptr)});
                return mm.add_literal(migraphx::literal{dense.get_shape(), dense.data()});
            },
            py::arg("data"))
        .def(
            "add_parameter",
            [](migraphx::module& mm, const std::string& name, const shape& s) { return mm.add_parameter(name, s); },
            py::arg("name"),
            py::arg("shape"))
        .def(
            "add_return",
            [](migraphx::module& mm, std::vector<instruction_ref>& args) { return mm.add_return(args); },
            py::arg("args"))
        .def("__repr__", [](const migraphx::module& mm) { return to_string(mm); });

    py::class_<migraphx::program>(m, "program")
        .def(py::init([] { return migraphx::program(); }))
        .def("get_parameter_names", &migraphx::program::get_parameter_names)
        .def("get_parameter_shapes", &migraphx::program::get_parameter_shapes)
        .def("get_output_shapes", &migraphx::program::get_output_shapes)
        .def("is_compiled", &migraphx::program::is_compiled)
        .def(
            "compile",
            [](migraphx::program& p, const migraphx::target& t, bool offload_copy, bool, bool) {
                migraphx::compile_options options;
                options.offload_copy = offload_copy;
                p.compile(t, options);
            },
            py::arg("t"),
            py::arg("offload_copy")    = true,
            py::arg("fast_math")       = true,
            py::arg("exhaustive_tune") = false)
        .def("get_main_module", [](migraphx::program& p) { return p.get_main_module(); },
             py::return_value_policy::reference_internal)
        .def("run",
             [](migraphx::program& p, const py::dict& params) {
                 auto r = p.eval(to_parameter_map(params));
                 p.finish();
                 return r;
             })
        .def("print", [](const migraphx::program& p) { std::cout << p << std::endl; })
        .def("__eq__", [](const migraphx::program& a, const migraphx::program& b) { return a == b; })
        .def("__ne__", [](const migraphx::program& a, const migraphx::program& b) { return a != b; })
        .def("__repr__", [](const migraphx::program& p) { return to_string(p); });

    // src/py/migraphx_py.cpp:699-760 (static shapes; the keyword arguments for dynamic shapes and
    // default dimensions are not part of this build)
    m.def("parse_onnx", [](const std::string& filename) { return migraphx::parse_onnx(filename); },
          "Parse onnx file", py::arg("filename"));
    m.def("parse_onnx_buffer",
          [](const py::bytes& buffer) { return migraphx::parse_onnx_buffer(std::string(buffer)); },
          "Parse onnx file from a buffer", py::arg("onnx_buffer"));
    // programs on disk (src/py/migraphx_py.cpp:753-793)
    m.def(
        "load",
        [](const std::string& filename, const std::string& format) {
            migraphx::file_options o;
            o.format = format;
            return migraphx::load(filename, o);
        },
        "Load MIGraphX program", py::arg("filename"), py::arg("format") = "msgpack");
    m.def(
        "save",
        [](const migraphx::program& p, const std::string& filename, const std::string& format) {
            migraphx::file_options o;
            o.format = format;
            migraphx::save(p, filename, o);
        },
        "Save MIGraphX program", py::arg("p"), py::arg("filename"), py::arg("format") = "msgpack");
    m.def(
        "save_buffer",
        [](const migraphx::program& p) {
            auto buffer = migraphx::save_buffer(p);
            return py::bytes(buffer.data(), buffer.size());
        },
        "Serialize MIGraphX program", py::arg("p"));
    m.def(
        "load_buffer",
        [](const py::bytes& b) {
            const std::string bytes = b;
            return migraphx::load_buffer(bytes.data(), bytes.size());
        },
        "Deserialize MIGraphX program", py::arg("b"));
    m.def("get_target", &get_target);
    m.def("create_argument", [](const shape& s, const std::vector<double>& values) {
        if(values.size() != s.elements())
            MIGRAPHX_THROW("Values and shape elements do not match");
        return argument{shape{s.type(), s.lens()}, values};
    });
    m.def(
        "quantize_int8",
        [](migraphx::program& prog, const migraphx::target& t, const std::vector<py::dict>& calibration,
           const std::unordered_set<std::string>& ins_names) {
            std::vector<migraphx::parameter_map> maps;
            for(const auto& d : calibration)
                maps.push_back(to_parameter_map(d));
            migraphx::quantize_int8(prog, t, maps, ins_names);
        },
        py::arg("prog"),
        py::arg("t"),
        py::arg("calibration") = std::vector<py::dict>{},
        py::arg("ins_names")   = std::unordered_set<std::string>{"dot", "convolution"});
    m.def(
        "quantize_fp8",
        [](migraphx::program& prog, const migraphx::target& t, const std::vector<py::dict>& calibration) {
            std::vector<migraphx::parameter_map> maps;
            for(const auto& d : calibration)
                maps.push_back(to_parameter_map(d));
            migraphx::quantize_fp8(prog, t, maps);
        },
        py::arg("prog"),
        py::arg("t"),
        py::arg("calibration") = std::vector<py::dict>{});
    // weight-only int4 (src/quantize_int4.cpp; `quantize_int4_weights` of src/include/migraphx/quantization.hpp)
    m.def("quantize_int4_weights", &migraphx::quantize_int4_weights, py::arg("prog"));

    m.def("allocate_gpu", [](const shape& s, bool) { return migraphx::mi355::allocate_device(s); }, py::arg("s"),
          py::arg("host") = false);
    m.def("to_gpu", [](const argument& a, bool) { return migraphx::mi355::to_device(a); }, py::arg("arg"),
          py::arg("host") = false);
    m.def("from_gpu", [](const argument& a) { return migraphx::mi355::from_device(a); });
}
