"""The Python surface of the host layer (`amdmigraphx_amd.migraphx`), checked on the CPU against the
behaviour of the reference's module (src/py/migraphx_py.cpp:362-626): construction of shapes,
operators, modules and programs, the buffer protocol of arguments, error reporting."""
import numpy as np
import pytest

mgx = pytest.importorskip("amdmigraphx_amd.migraphx")


def test_shape_constructor_keywords():
    s = mgx.shape(type="float", lens=[4, 8])
    assert s.lens() == [4, 8] and s.strides() == [8, 1] and s.standard() and s.elements() == 32
    assert s.type() == mgx.shape.type_t.float_type and s.type_string() == "float_type" and s.type_size() == 4
    assert mgx.shape().lens() == [1] and mgx.shape().type_string() == "float_type"   # the defaults
    t = mgx.shape(type="int8", lens=[2, 3], strides=[1, 2])
    assert t.transposed() and not t.standard() and t.bytes() == 6
    p = mgx.shape(type="half", lens=[2, 3, 4], permutation=[0, 2, 1])
    assert p.lens() == [2, 3, 4] and p.strides() == [12, 1, 3]
    assert mgx.shape(type="int32", lens=[5]) == mgx.shape(type="int32", lens=[5])
    assert mgx.shape(type="int32", lens=[5]) != mgx.shape(type="float", lens=[5])
    assert repr(s) == "float_type, {4, 8}, {8, 1}"
    with pytest.raises(RuntimeError):
        mgx.shape(type="no_such_type", lens=[1])


def test_operator_attributes():
    op = mgx.op("quant_convolution", padding=[1, 1], stride=[2, 2])
    assert op.name() == "quant_convolution"
    assert op.values() == {"padding": [1, 1], "stride": [2, 2], "dilation": [1, 1], "padding_mode": 0, "group": 1}
    assert mgx.op("transpose", permutation=(1, 0)).values() == {"permutation": [1, 0]}
    assert mgx.op("convert", target_type=mgx.shape.type_t.half_type).values()["target_type"] == \
        int(mgx.shape.type_t.half_type)
    with pytest.raises(RuntimeError):
        mgx.op("transpose", no_such_attribute=1)
    with pytest.raises(RuntimeError):
        mgx.op("no_such_operator")


def build_matmul(k=8, n=4):
    p = mgx.program()
    mm = p.get_main_module()
    x = mm.add_parameter("x", mgx.shape(type="float", lens=[4, k]))
    w = mm.add_literal(np.arange(k * n, dtype=np.float32).reshape(k, n))
    d = mm.add_instruction(mgx.op("dot"), [x, w])
    mm.add_return([d])
    return p, d


def test_program_construction_and_printing():
    p, d = build_matmul()
    assert p.get_parameter_names() == ["x"]
    assert p.get_parameter_shapes()["x"] == mgx.shape(type="float", lens=[4, 8])
    assert p.get_output_shapes() == [mgx.shape(type="float", lens=[4, 4])]
    assert not p.is_compiled()
    assert d.name() == "dot" and d.shape().lens() == [4, 4]
    assert [i.name() for i in d.inputs()] == ["@param", "@literal"]
    assert [o.name() for o in d.outputs()] == ["@return"]
    text = repr(p)
    assert "dot(" in text and "@param:x" in text and "@return" in text
    q, _ = build_matmul()
    assert p == q
    r, _ = build_matmul(n=5)
    assert p != r
    # shape errors of an operator surface as Python exceptions with the operator's message
    mm = p.get_main_module()
    with pytest.raises(RuntimeError, match="DOT"):
        mm.add_instruction(mgx.op("dot"), [d, d.inputs()[1]])


def test_argument_buffer_protocol():
    a = np.arange(24, dtype=np.int32).reshape(2, 3, 4)
    arg = mgx.argument(a)
    assert arg.get_shape() == mgx.shape(type="int32", lens=[2, 3, 4])
    assert np.array_equal(np.array(arg), a) and arg.tolist() == list(map(float, range(24)))
    # a transposed view is taken element by element
    t = mgx.argument(a.transpose(2, 0, 1))
    assert t.get_shape().lens() == [4, 2, 3] and np.array_equal(np.array(t), a.transpose(2, 0, 1))
    h = mgx.argument(np.float16([1.5, -2.0]))
    assert h.get_shape().type_string() == "half_type" and h.tolist() == [1.5, -2.0]
    assert arg == mgx.argument(a.copy()) and arg != mgx.argument(a + 1)
    c = mgx.create_argument(mgx.shape(type="int8", lens=[3]), [1, -2, 3])
    assert np.array(c).dtype == np.int8 and np.array(c).tolist() == [1, -2, 3]
    with pytest.raises(RuntimeError):
        mgx.create_argument(mgx.shape(type="int8", lens=[3]), [1, 2])


def test_literals_keep_their_element_type():
    p = mgx.program()
    mm = p.get_main_module()
    for dt, name in ((np.int8, "int8_type"), (np.uint8, "uint8_type"), (np.float16, "half_type"),
                     (np.int32, "int32_type"), (np.int64, "int64_type")):
        lit = mm.add_literal(np.ones((2, 2), dt))
        assert lit.shape().type_string() == name and lit.name() == "@literal"


def test_weight_only_int4_quantization_pass():
    # src/quantize_int4.cpp:38-103: the constant operand of a dot is packed to int4 behind
    # unpack_int4 + dequantizelinear
    p = mgx.program()
    mm = p.get_main_module()
    x = mm.add_parameter("x", mgx.shape(type="half", lens=[1, 256]))
    w = mm.add_literal((np.random.default_rng(0).standard_normal((256, 64)) * 0.1).astype(np.float16))
    mm.add_return([mm.add_instruction(mgx.op("dot"), [x, w])])
    mgx.quantize_int4_weights(p)
    text = repr(p)
    assert "unpack_int4" in text and "dequantizelinear" in text


def test_targets():
    assert mgx.get_target("gpu").name() == "mi355"      # the reference's name for the device target
    assert mgx.get_target("mi355").name() == "mi355"
    with pytest.raises(RuntimeError):
        mgx.get_target("no_such_target")


def quantized_matmul_program():
    p, _ = build_matmul(k=256, n=64)
    mgx.quantize_int4_weights(p)
    return p


def test_save_and_load(tmp_path):
    # src/py/migraphx_py.cpp:753-793: load / save with a format keyword, save_buffer / load_buffer
    p = quantized_matmul_program()
    for fmt in ("msgpack", "json"):
        name = str(tmp_path / ("prog." + fmt))
        mgx.save(p, name, format=fmt)
        q = mgx.load(name, format=fmt)
        assert q == p and repr(q) == repr(p)
    name = str(tmp_path / "default.mxr")
    mgx.save(p, name)
    assert mgx.load(name) == p
    buf = mgx.save_buffer(p)
    assert isinstance(buf, bytes) and open(name, "rb").read() == buf
    assert mgx.load_buffer(buf) == p
    with pytest.raises(RuntimeError):
        mgx.load(str(tmp_path / "missing.mxr"))
    with pytest.raises(RuntimeError):
        mgx.save(p, str(tmp_path / "x"), format="yaml")
    with pytest.raises(RuntimeError):
        mgx.load_buffer(buf[: len(buf) // 2])


def test_saved_program_is_standard_messagepack():
    """The saved bytes are checked against an independent MessagePack implementation (the `msgpack`
    Python package): it decodes them to the fields src/program.cpp:720-777 writes, re-encoding what
    it decoded gives the same bytes (every number and length is in its shortest form), and bytes it
    encodes load as the same program."""
    msgpack = pytest.importorskip("msgpack")
    p = quantized_matmul_program()
    buf = mgx.save_buffer(p)
    doc = msgpack.unpackb(buf, raw=False, strict_map_key=True)
    assert doc["version"] == 8 and isinstance(doc["migraphx_version"], str)
    assert doc["targets"] == [] and doc["contexts"] == []
    assert list(doc["modules"]) == ["main"] and doc["modules"]["main"]["name"] == "main"
    nodes = doc["modules"]["main"]["nodes"]
    assert [n["name"] for n in nodes].count("@literal") >= 2          # packed weights and scales
    by_output = {n["output"]: n for n in nodes}
    assert len(by_output) == len(nodes)
    for i, n in enumerate(nodes):
        assert set(n) >= {"output", "name", "shape", "normalized", "operator", "inputs"}
        assert n["output"] == (n["operator"]["parameter"] if n["name"] == "@param" else "@%d" % i)
        assert all(j in by_output for j in n["inputs"])
        assert set(n["shape"]) == {"type", "sub_shapes", "lens", "strides", "dynamic_dimensions", "dyn_strides"}
    x = by_output["x"]
    assert x["shape"]["type"] == "float_type" and x["shape"]["lens"] == [4, 256]
    lit = next(n for n in nodes if n["name"] == "@literal" and n["shape"]["type"] == "uint8_type")
    data = lit["literal"]["data"]
    # binary data is an array of bin chunks
    assert isinstance(data, list) and len(data) == 1 and isinstance(data[0], bytes)
    assert len(data[0]) == int(np.prod(lit["shape"]["lens"]))
    unpack = next(n for n in nodes if n["name"] == "unpack_int4")
    assert unpack["operator"] == {"axis": -1}
    assert msgpack.packb(doc, use_bin_type=True) == buf
    assert mgx.load_buffer(msgpack.packb(doc, use_bin_type=True)) == p
    # an edit made outside survives the trip: rename the parameter
    for n in nodes:
        if n["name"] == "@param":
            n["output"] = n["operator"]["parameter"] = "activations"
        n["inputs"] = ["activations" if j == "x" else j for j in n["inputs"]]
    q = mgx.load_buffer(msgpack.packb(doc, use_bin_type=True))
    assert q.get_parameter_names() == ["activations"] and q.get_output_shapes() == p.get_output_shapes()
    # JSON form: standard JSON with the same fields
    import json
    name_json = json.loads(open_json(p))
    assert name_json["version"] == 8 and [n["name"] for n in name_json["modules"]["main"]["nodes"]] == \
        [n["name"] for n in nodes]
    jl = next(n for n in name_json["modules"]["main"]["nodes"]
              if n["name"] == "@literal" and n["shape"]["type"] == "uint8_type")
    assert bytes(jl["literal"]["data"]["bytes"]) == data[0]


def open_json(p):
    import os
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        name = os.path.join(d, "p.json")
        mgx.save(p, name, format="json")
        return open(name).read()
