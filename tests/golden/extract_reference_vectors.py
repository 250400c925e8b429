#!/usr/bin/env python3
"""Collect the known-answer vectors that the reference's own tests hold for the
quantized-GEMM path and write them to ``reference_vectors.json``.

Run in the build container only (it reads the reference tree as text):

    python tests/golden/extract_reference_vectors.py [/root/reference]

The output holds DATA only: literal inputs, shapes, attributes and expected
outputs of the reference's test cases, each tagged with the file it was read
from.  No reference code is executed, imported or stored.
"""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")


def read(rel):
    with open(os.path.join(REF, rel)) as f:
        return f.read()


def num(tok):
    t = tok.strip().replace("'", "")
    t = re.sub(r"/\*.*?\*/", "", t).strip()
    if not t:
        return None
    if "quiet_NaN" in t:
        return "nan"
    if "infinity" in t:
        return "-inf" if t.startswith("-") else "inf"
    neg = t.startswith("-")
    if neg:
        t = t[1:]
    if t.lower().startswith("0x"):
        v = int(t, 16)
    elif t.lower().startswith("0b"):
        v = int(t, 2)
    else:
        t = t.rstrip("fF")
        v = float(t) if any(c in t for c in ".eE") else int(t)
    return -v if neg else v


def num_list(s):
    s = re.sub(r"/\*.*?\*/", "", s, flags=re.S)
    s = re.sub(r"//[^\n]*", "", s)
    return [v for v in (num(t) for t in s.split(",")) if v is not None]


def test_cases(text):
    """name -> body for every TEST_CASE(name) { ... } (bodies end at the next
    TEST_CASE / template / EOF, which is enough for vector scraping)."""
    out = {}
    marks = [(m.start(), m.group(1)) for m in re.finditer(r"TEST_CASE\((\w+)\)", text)]
    cuts = sorted([p for p, _ in marks] +
                  [m.start() for m in re.finditer(r"\ntemplate <", text)] + [len(text)])
    for pos, name in marks:
        end = min(c for c in cuts if c > pos)
        out[name] = text[pos:end]
    return out


def vec(body, name):
    m = re.search(r"\b" + re.escape(name) + r"\s*(?:=\s*)?\{(.*?)\};", body, re.S)
    if not m:
        return None
    return num_list(m.group(1))


def shape(body, name):
    m = re.search(r"(?:migraphx::shape\s+" + re.escape(name) + r"|auto " + re.escape(name) +
                  r"\s*=\s*migraphx::shape)"
                  r"\{migraphx::shape::(\w+)_type,\s*\{([^}]*)\}(?:,\s*\{([^}]*)\})?\}", body)
    if not m:
        return None
    d = {"type": m.group(1), "lens": num_list(m.group(2))}
    if m.group(3):
        d["strides"] = num_list(m.group(3))
    return d


out = {"_provenance": "literal inputs and expected outputs read from the reference's test sources"}

# ---- fp8 e4m3fn table and cast samples (test/fp8e4m3fn.cpp) ------------------
t = read("test/fp8e4m3fn.cpp")
m = re.search(r"e4m3fnuz_lut = \{(.*?)\};", t, re.S)
out["fp8e4m3fn_lut"] = {"source": "test/fp8e4m3fn.cpp:34-105", "values": num_list(m.group(1))}
m = re.search(r"test_vals = \{\s*\{(.*?)\}\};", t, re.S)
pairs = re.findall(r"\{\s*([-+0-9.eE]+)\s*,\s*(0x[0-9a-fA-F]+)\s*\}", m.group(1))
out["fp8e4m3fn_from_float"] = {"source": "test/fp8e4m3fn.cpp:121-140",
                               "pairs": [[float(a), int(b, 16)] for a, b in pairs]}

# ---- fp8 e5m2 table and cast samples (test/fp8e5m2.cpp) ----------------------
t = read("test/fp8e5m2.cpp")
m = re.search(r"e4m3fnuz_lut = \{(.*?)\};", t, re.S)     # (the table keeps that name in this file too)
out["fp8e5m2_lut"] = {"source": "test/fp8e5m2.cpp:37-295", "values": num_list(m.group(1))}
m = re.search(r"test_vals = \{\s*\{(.*?)\}\s*,?\s*\};", t, re.S)
pairs = re.findall(r"\{\s*([-+0-9.eE]+)\s*,\s*(0x[0-9a-fA-F]+)\s*\}", "{" + m.group(1) + "}")
out["fp8e5m2_from_float"] = {"source": "test/fp8e5m2.cpp:320-360",
                             "pairs": [[float(a), int(b, 16)] for a, b in pairs]}

# ---- half / bf16 tables ------------------------------------------------------
for nm, rel in (("half", "test/half.cpp"), ("bf16", "test/bf16.cpp")):
    t = read(rel)
    m = re.search(nm + r"_lut\(\).*?result = \{(.*?)\n    \};", t, re.S)
    pairs = re.findall(r"\{\s*(0x[0-9a-fA-F]+)\s*,\s*([^}]+)\}", m.group(1))
    out[nm + "_lut"] = {"source": rel, "pairs": [[int(a, 16), num(b)] for a, b in pairs]}

# ---- quant_dot known answers (test/ref/dot_op.cpp) -----------------------------
t = read("test/ref/dot_op.cpp")
cases = test_cases(t)
qd = []
for name, body in cases.items():
    if not name.startswith("quant_dot_") or "4args" in name:
        continue
    c = {"name": name, "source": "test/ref/dot_op.cpp"}
    c["a"] = shape(body, "m1_shape")
    c["b"] = shape(body, "m2_shape")
    c["c"] = shape(body, "m3_shape")
    c["a_perm"] = None
    c["b_perm"] = None
    m1 = re.search(r"auto tl1\s*=\s*mm->add_instruction\(\s*migraphx::make_op\(\"transpose\", "
                   r"\{\{\"permutation\", \{([^}]*)\}\}\}\),\s*l1\)", body, re.S)
    m2 = re.search(r"auto tl2\s*=\s*mm->add_instruction\(\s*migraphx::make_op\(\"transpose\", "
                   r"\{\{\"permutation\", \{([^}]*)\}\}\}\),\s*l2\)", body, re.S)
    if m1:
        c["a_perm"] = num_list(m1.group(1))
    if m2:
        c["b_perm"] = num_list(m2.group(1))
    ab = re.search(r"add_apply_alpha_beta\(\s*\*mm,\s*\{([^}]*)\},\s*migraphx::make_op\(\"quant_dot\"\)"
                   r"(?:,\s*([-0-9.]+))?(?:,\s*([-0-9.]+))?\)", body, re.S)
    c["alpha"], c["beta"], c["uses_c"] = 1, 0, False
    if ab:
        args = [a.strip() for a in ab.group(1).split(",")]
        c["uses_c"] = len(args) == 3
        if ab.group(2):
            c["alpha"] = num(ab.group(2))
        if ab.group(3):
            c["beta"] = num(ab.group(3))
    c["iota_start"] = {"a": 0, "b": 0}
    m3 = re.search(r"std::iota\(data3\.begin\(\), data3\.end\(\), (\d+)\)", body)
    if m3:
        c["iota_start"]["c"] = int(m3.group(1))
    c["gold"] = vec(body, "gold")
    qd.append(c)
out["quant_dot"] = qd

body = cases["quant_dot_4args_scales"]
out["quant_dot_4args_scales"] = {
    "source": "test/ref/dot_op.cpp", "a": vec(body, "a_data"), "b": vec(body, "b_data"),
    "scale_a": vec(body, "scale_a_data"), "scale_b": vec(body, "scale_b_data"),
    "a_lens": [2, 3], "b_lens": [3, 2], "gold": vec(body, "gold")}

# ---- quantizelinear / dequantizelinear -----------------------------------------
t = read("test/ref/quantizelinear.cpp")
cases = test_cases(t)
ql = []
for name in ("quantizelinear_1", "quantizelinear_2"):
    body = cases[name]
    ql.append({"name": name, "source": "test/ref/quantizelinear.cpp", "x": vec(body, "xv"),
               "scale": vec(body, "sv"), "zp": vec(body, "zv"),
               "zp_type": (shape(body, "zs") or {}).get("type"),
               "lens": shape(body, "xs")["lens"], "gold": vec(body, "gold")})
out["quantizelinear"] = ql
m = re.search(r"static void quantizelinear_fp8e4m3\(\)(.*?)TEST_CASE_REGISTER", t, re.S)
body = m.group(1)
out["quantizelinear_fp8e4m3"] = {
    "source": "test/ref/quantizelinear.cpp:86-127 (gold is computed there as "
              "fp8(clamp(x/s + fp8(zp))) in double)",
    "x": vec(body, "xv"), "scale": vec(body, "sv"), "zp_float": vec(body, "tmp"), "lens": [2, 2, 2]}
m = re.search(r"static void quantizelinear_fp8e5m2\(\)(.*?)TEST_CASE_REGISTER", t, re.S)
body = m.group(1)
out["quantizelinear_fp8e5m2"] = {
    "source": "test/ref/quantizelinear.cpp:129-168 (gold is computed there as "
              "fp8(clamp(x/s) + fp8(zp)) in double)",
    "x": vec(body, "xv"), "scale": vec(body, "sv"), "zp_float": vec(body, "tmp"), "lens": [2, 2, 2]}

t = read("test/ref/dequantizelinear.cpp")
cases = test_cases(t)
dq = []
for name, body in cases.items():
    dq.append({"name": name, "source": "test/ref/dequantizelinear.cpp", "x": vec(body, "xv"),
               "x_type": shape(body, "xs")["type"], "scale": vec(body, "sv"), "zp": vec(body, "zv"),
               "lens": shape(body, "xs")["lens"], "gold": vec(body, "gold")})
out["dequantizelinear"] = dq

# ---- unpack_int4 / pack_int4 -----------------------------------------------------
def int4_cases(rel, opname):
    t = read(rel)
    res = []
    for name, body in test_cases(t).items():
        s = shape(body, "s")
        lit = re.search(r"migraphx::literal\{\s*s,\s*\{(.*?)\}\}", body, re.S)
        if not s or not lit:
            continue
        c = {"name": name, "source": rel, "shape": s, "data": num_list(lit.group(1)),
             "gold": vec(body, "gold")}
        ax = re.search(r"make_op\(\"" + opname + r"\", \{\{\"axis\", (-?\d+)\}\}\)", body)
        c["axis"] = int(ax.group(1)) if ax else -1
        mb = re.search(r"multibroadcast\", \{\{\"out_lens\", \{([^}]*)\}\}\}", body)
        c["multibroadcast"] = num_list(mb.group(1)) if mb else None
        res.append(c)
    return res


out["unpack_int4"] = int4_cases("test/ref/unpack_int4.cpp", "unpack_int4")
out["pack_int4"] = int4_cases("test/ref/pack_int4.cpp", "pack_int4")

# ---- MatMulNBits end-to-end golds (test/onnx/verify/matmulnbits_tests.cpp) -------
# N, K and block size are fixed by the tensor shapes: b is [N, ceil(K/blk), blk/2]
# (src/onnx/parse_matmulnbits.cpp:60-66) and K is a's last dimension.
t = read("test/onnx/verify/matmulnbits_tests.cpp")
mn = []
for name, body in test_cases(t).items():
    c = {"name": name, "source": "test/onnx/verify/matmulnbits_tests.cpp",
         "a_lens": shape(body, "a_shape")["lens"], "b_lens": shape(body, "b_shape")["lens"]}
    m = re.search(r"std::vector<float> a\{(.*?)\};", body, re.S)
    c["a"] = num_list(m.group(1)) if m else "iota"
    c["b"] = vec(body, "b")
    c["scales"] = vec(body, "scales")
    c["zp"] = vec(body, "zp") if "zp_shape" in body else None
    c["gold"] = vec(body, "gold")
    mn.append(c)
out["matmulnbits"] = mn

# ---- float operators of the encoder graph: softmax, reduce_mean, gather ----------------------
t = read("test/ref/softmax.cpp")
cases = test_cases(t)
sm = []
for name in ("softmax_simple_test", "softmax_test"):
    body = cases[name]
    ax = int(re.search(r'"softmax",\s*\{\{"axis",\s*(-?\d+)\}\}', body).group(1))
    sm.append({"name": name, "source": "test/ref/softmax.cpp", "shape": shape(body, "a_shape"),
               "axis": ax, "a": vec(body, "a"), "gold": vec(body, "gold")})
out["softmax"] = sm

t = read("test/ref/reduce_mean.cpp")
cases = test_cases(t)
rm = []
for name in ("reduce_mean_axis02", "reduce_mean_axis1", "reduce_mean_axis12", "reduce_mean_axis2"):
    body = cases[name]
    axes = num_list(re.search(r'"reduce_mean",\s*\{\{"axes",\s*\{([^}]*)\}\}\}', body).group(1))
    inp = num_list(re.search(r"migraphx::literal\{s,\s*\{([^}]*)\}\}", body).group(1))
    rm.append({"name": name, "source": "test/ref/reduce_mean.cpp", "shape": shape(body, "s"),
               "axes": axes, "input": inp, "gold": vec(body, "gold")})
out["reduce_mean"] = rm

t = read("test/ref/gather.cpp")
cases = test_cases(t)
ga = []
for i in range(1, 8):
    body = cases["gather_test_%d" % i]
    n = num_list(re.search(r"std::vector<float> data\(([^)]*)\)", body).group(1).replace("*", ","))
    count = 1
    for v in n:
        count *= v
    sidx = re.search(r"migraphx::shape s_indices\{migraphx::shape::int32_type(?:,\s*\{([^}]*)\})?\}", body)
    ga.append({"name": "gather_test_%d" % i, "source": "test/ref/gather.cpp",
               "data_iota_start": 0.5, "data_count": count, "shape": shape(body, "s"),
               "indices_lens": num_list(sidx.group(1)) if sidx.group(1) else None,
               "indices": vec(body, "indices"),
               "axis": int(re.search(r"int axis\s*=\s*(-?\d+);", body).group(1)),
               "gold": vec(body, "golden")})
out["gather"] = ga

# ---- pack_fp4 / unpack_fp4 (test/ref/pack_unpack_fp4.cpp) ---------------------------
t = read("test/ref/pack_unpack_fp4.cpp")
cases = test_cases(t)
fp4 = []
body = cases["pack_fp4"]
fp4.append({"name": "pack_fp4", "source": "test/ref/pack_unpack_fp4.cpp",
            "lens": num_list(re.search(r"float_type,\s*\{([^}]*)\}", body).group(1)),
            "input": num_list(re.search(r"migraphx::literal\{s,\s*\{([^}]*)\}\}", body).group(1)),
            "axis": int(re.search(r'"axis",\s*(-?\d+)', body).group(1)),
            "gold_bytes": num_list(re.search(r"std::vector<uint8_t> gold\{([^}]*)\}", body).group(1))})
body = cases["unpack_fp4"]
fp4.append({"name": "unpack_fp4", "source": "test/ref/pack_unpack_fp4.cpp",
            "lens": num_list(re.search(r"fp4x2_type,\s*\{([^}]*)\}", body).group(1)),
            "input_bytes": num_list(re.search(r"packed_data\s*=\s*\{([^}]*)\}", body).group(1)),
            "axis": int(re.search(r'"axis",\s*(-?\d+)', body).group(1)),
            "gold": num_list(re.search(r"std::vector<float> gold\{([^}]*)\}", body).group(1))})
body = cases["pack_unpack_fp4"]
fp4.append({"name": "pack_unpack_fp4", "source": "test/ref/pack_unpack_fp4.cpp",
            "lens": num_list(re.search(r"float_type,\s*\{([^}]*)\}", body).group(1)),
            "input": num_list(re.search(r"migraphx::literal\{s,\s*\{([^}]*)\}\}", body).group(1)),
            "axis": int(re.search(r'"axis",\s*(-?\d+)', body).group(1)),
            "gold": num_list(re.search(r"std::vector<float> gold\{([^}]*)\}", body).group(1))})
out["fp4"] = fp4

# ---- convolution known answers (test/ref/quant_convolution.cpp, convolution.cpp) ---------------
def conv_attrs(body, opname):
    m = re.search(r'make_op\(\s*"' + opname + r'"\s*(?:,\s*\{(.*?)\}\s*)?\)\s*,\s*al', body, re.S)
    attrs = {"padding": [0, 0], "stride": [1, 1], "dilation": [1, 1], "group": 1}
    if m and m.group(1):
        for key in ("padding", "stride", "dilation"):
            k = re.search(r'"' + key + r'",\s*\{([^}]*)\}', m.group(1))
            if k:
                attrs[key] = num_list(k.group(1))
        g = re.search(r'"group",\s*(\d+)', m.group(1))
        if g:
            attrs["group"] = int(g.group(1))
    return attrs


conv = []
cases = test_cases(read("test/ref/quant_convolution.cpp"))
for name in ("quant_conv2d_test", "quant_conv2d_padding_test", "quant_conv2d_padding_stride_test"):
    body = cases[name]
    c = {"name": name, "source": "test/ref/quant_convolution.cpp", "type": "int8",
         "x_lens": shape(body, "a_shape")["lens"], "w_lens": shape(body, "c_shape")["lens"],
         "x": "iota", "w": "iota", "gold": vec(body, "gold")}
    c.update(conv_attrs(body, "quant_convolution"))
    conv.append(c)
cases = test_cases(read("test/ref/convolution.cpp"))
body = cases["conv2d_dilation_test"]
c = {"name": "conv2d_dilation_test", "source": "test/ref/convolution.cpp:674-701", "type": "float",
     "x_lens": shape(body, "a_shape")["lens"], "w_lens": shape(body, "c_shape")["lens"],
     "x": "iota", "w": "iota", "gold": vec(body, "gold")}
c.update(conv_attrs(body, "convolution"))
conv.append(c)
body = cases["conv2d_grouped_test"]
c = {"name": "conv2d_grouped_test", "source": "test/ref/convolution.cpp:761-857", "type": "float",
     "x_lens": shape(body, "a_shape")["lens"], "w_lens": shape(body, "c_shape")["lens"],
     "x": vec(body, "a"), "w": vec(body, "c"), "gold": vec(body, "gold")}
c.update(conv_attrs(body, "convolution"))
conv.append(c)
# three spatial axes: the float operator's known answers pin the loop order and the indexing of
# the shared convolution routine (quant_convolution calls the same one)
for name, where in (("conv3d_test", "test/ref/convolution.cpp:991-1060"),
                    ("conv3d_grouped_test", "test/ref/convolution.cpp:859-989")):
    body = cases[name]
    c = {"name": name, "source": where, "type": "float",
         "x_lens": shape(body, "a_shape")["lens"], "w_lens": shape(body, "c_shape")["lens"],
         "x": vec(body, "a"), "w": vec(body, "c"), "gold": vec(body, "gold")}
    c.update(conv_attrs(body, "convolution"))
    conv.append(c)
out["convolution"] = conv

# ---- ONNX Q/DQ models with their expected outputs (test/onnx/verify/*_blocked_test.cpp) ---------
onnx_cases = []
for rel in ("test/onnx/verify/dequantizelinear_blocked_test.cpp", "test/onnx/verify/quantizelinear_blocked_test.cpp"):
    for name, body in test_cases(read(rel)).items():
        model = re.search(r'read_onnx\("([^"]+)"\)', body).group(1)
        c = {"name": name, "source": rel, "model": model, "inputs": {}}
        # pm["<parameter>"] = migraphx::argument{<var>_shape, <var>.data()};
        for param, var in re.findall(r'pm\["(\w+)"\]\s*=\s*migraphx::argument\{\w+,\s*(\w+)\.data\(\)\}', body):
            c["inputs"][param] = vec(body, var)
        c["gold"] = vec(body, "gold")
        onnx_cases.append(c)
out["onnx_qdq"] = onnx_cases

# ---- QLinearMatMul models (test/onnx/verify/qlinearmatmul_*_test.cpp, QLinearMatMul_2d_per_channel_test.cpp)
qlm = []
for rel in ("test/onnx/verify/qlinearmatmul_1D_test.cpp", "test/onnx/verify/qlinearmatmul_2D_test.cpp",
            "test/onnx/verify/qlinearmatmul_3D_test.cpp", "test/onnx/verify/qlinearmatmul_N_D_perchannel_test.cpp",
            "test/onnx/verify/QLinearMatMul_2d_per_channel_test.cpp"):
    for name, body in test_cases(read(rel)).items():
        model = re.search(r'read_onnx\("([^"]+)"\)', body).group(1)
        c = {"name": name, "source": rel, "model": model, "inputs": {}}
        for param, var in re.findall(r'pp\["(\w+)"\]\s*=\s*migraphx::argument\(\w+,\s*(\w+)\.data\(\)\)', body):
            c["inputs"][param] = vec(body, var)
        c["gold"] = vec(body, "gold")
        # the 2-D per-channel case builds its input in code and its model holds a 2 MB weight: left out
        if any(v is None for v in c["inputs"].values()):
            continue
        qlm.append(c)
out["onnx_qlinearmatmul"] = qlm

# ---- integer MatMul / QLinearConv models (test/onnx/verify/matmulinteger*_test.cpp, qlinearconv_*_test.cpp)
ints = []
for stem in ("matmulinteger_int8_uint8_test", "matmulinteger_int8_uint8_one_zp_test",
             "matmulinteger_int8_uint8_dual_zp_test", "matmulinteger_uns_test", "matmulinteger_uns_zp_test",
             "matmulintegertofloat_int8_uint8_scales_zp_bias", "matmulintegertofloat_int8_uint8_scales_zp_bias_3d",
             "qlinearconv_test", "qlinearconv_pad_0_test", "qlinearconv_pad_1_test", "qlinearconv_scale_1D_test",
             "qlinearconv_perchannel_weightbias_test"):
    rel = "test/onnx/verify/" + stem + ".cpp"
    for name, body in test_cases(read(rel)).items():
        model = re.search(r'read_onnx\("([^"]+)"\)', body).group(1)
        c = {"name": name, "source": rel, "model": model, "inputs": {}}
        for param, var in re.findall(r'pp\["(\w+)"\]\s*=\s*migraphx::argument\(\w+,\s*(\w+)\.data\(\)\)', body):
            v = vec(body, var)
            if v is None and re.search(r"std::iota\(" + var + r"\.begin\(\)", body):
                # std::vector<T> var(shape.elements(), 0); std::iota(...): 0, 1, 2, ...
                shp = re.search(r"std::vector<\w+>\s+" + var + r"\((\w+)\.elements\(\)", body).group(1)
                n = 1
                for d in shape(body, shp)["lens"]:
                    n *= d
                v = list(range(n))
            if v is None and re.search(var + r"\[i\]\s*=\s*static_cast<uint8_t>\(i % 256\)", body):
                # for(i ...) var[i] = i % 256 over the whole tensor
                shp = re.search(r"std::vector<\w+>\s+" + var + r"\((\w+)\.elements\(\)\)", body).group(1)
                n = 1
                for d in shape(body, shp)["lens"]:
                    n *= d
                v = {"rule": "index mod 256", "count": n}
            c["inputs"][param] = v
        c["gold"] = vec(body, "gold")
        if c["gold"] is None:
            # only the first outputs are listed
            c["gold"] = vec(body, "gold_prefix")
            c["gold_is_prefix"] = True
        assert c["gold"] is not None and all(v is not None for v in c["inputs"].values()), name
        ints.append(c)
        # the model itself is a data file of the reference's tests: kept beside the vectors
        import shutil
        shutil.copyfile(os.path.join(REF, "test/onnx", model), os.path.join(os.path.dirname(OUT), "onnx", model))
out["onnx_integer"] = ints

# ---- DynamicQuantizeLinear models (test/onnx/verify/dynamicquantizelinear_{1d,2d}_test.cpp): three outputs
dql = []
for stem in ("dynamicquantizelinear_1d_test", "dynamicquantizelinear_2d_test"):
    rel = "test/onnx/verify/" + stem + ".cpp"
    for name, body in test_cases(read(rel)).items():
        model = re.search(r'read_onnx\("([^"]+)"\)', body).group(1)
        dql.append({"name": name, "source": rel, "model": model, "x": vec(body, "data"),
                    "y": vec(body, "y_gold"), "y_scale": vec(body, "y_scale_gold"), "y_zero_point": vec(body, "y_zpt_gold")})
        import shutil
        shutil.copyfile(os.path.join(REF, "test/onnx", model), os.path.join(os.path.dirname(OUT), "onnx", model))
out["onnx_dynamicquantizelinear"] = dql

# ---- MatMulBnb4 models (test/onnx/verify/matmulbnb4_tests.cpp): A, the packed 4-bit codes, absmax, result
bnb = []
rel = "test/onnx/verify/matmulbnb4_tests.cpp"
for name, body in test_cases(read(rel)).items():
    model = re.search(r'optimize_onnx\("([^"]+)"\)', body).group(1)
    c = {"name": name, "source": rel, "model": model, "inputs": {}}
    for param, var in re.findall(r'pm\["(\w+)"\]\s*=\s*migraphx::argument\(\w+,\s*(\w+)\.data\(\)\)', body):
        v = vec(body, var)
        if v is None:
            # std::vector<float> a(a_shape.elements()); std::iota(a.begin(), a.end(), start)
            start = num(re.search(r"std::iota\(" + var + r"\.begin\(\),\s*" + var + r"\.end\(\),\s*([^)]+)\)", body).group(1))
            n = 1
            for d in shape(body, var + "_shape")["lens"]:
                n *= d
            v = [start + i for i in range(n)]
        c["inputs"][param] = v
    c["gold"] = vec(body, "gold")
    c["lens"] = num_list(re.search(r"get_shape\(\)\.lens\(\) == std::vector<size_t>\{([^}]*)\}", body).group(1))
    assert c["gold"] is not None and all(v is not None for v in c["inputs"].values()), name
    bnb.append(c)
import glob
import shutil
for f in sorted(glob.glob(os.path.join(REF, "test/onnx", "matmulbnb4_*.onnx"))):
    shutil.copyfile(f, os.path.join(os.path.dirname(OUT), "onnx", os.path.basename(f)))
out["onnx_matmulbnb4"] = bnb

# ---- QLinearAdd / QLinearMul models (test/onnx/verify/qlinear{add,mul}[_bcast]_test.cpp): 8-bit results
qlb = []
for stem in ("qlinearadd_test", "qlinearadd_bcast_test", "qlinearmul_test", "qlinearmul_bcast_test"):
    rel = "test/onnx/verify/" + stem + ".cpp"
    for name, body in test_cases(read(rel)).items():
        model = re.search(r'read_onnx\("([^"]+)"\)', body).group(1)
        c = {"name": name, "source": rel, "model": model, "inputs": {}}
        for param, var in re.findall(r'pp\["(\w+)"\]\s*=\s*migraphx::argument\(\w+,\s*(\w+)\.data\(\)\)', body):
            c["inputs"][param] = vec(body, var)
        c["gold"] = vec(body, "gold")
        assert c["gold"] is not None and all(v is not None for v in c["inputs"].values()), name
        qlb.append(c)
        shutil.copyfile(os.path.join(REF, "test/onnx", model), os.path.join(os.path.dirname(OUT), "onnx", model))
out["onnx_qlinearbinary"] = qlb

# ---- LayerNormalization models (test/onnx/verify/layer_norm_3d*_test.cpp): x = 1, 2, 3, ... (norm_test in
# test/onnx/include/onnx_verify_utils.hpp:33-60), scale and bias as the test gives them
lnm = []
for stem in ("layer_norm_3d_test", "layer_norm_3d_half_test", "layer_norm_3d_bf16_test"):
    rel = "test/onnx/verify/" + stem + ".cpp"
    for name, body in test_cases(read(rel)).items():
        flat = re.sub(r"(?:half|bf16|migraphx::half|migraphx::bf16)\{([^}]*)\}", r"\1", body)
        call = re.search(r"norm_test<(\w+)>\(\{([^}]*)\},\s*scale,\s*bias,\s*read_onnx\(\"([^\"]+)\"\)", flat)
        c = {"name": name, "source": rel, "model": call.group(3), "type": call.group(1),
             "x_lens": num_list(call.group(2)), "scale": vec(flat, "scale"), "bias": vec(flat, "bias"),
             "gold": vec(flat, "gold")}
        assert c["gold"] and c["scale"] and c["bias"], name
        lnm.append(c)
for f in sorted(glob.glob(os.path.join(REF, "test/onnx", "layer_norm_*.onnx"))):
    shutil.copyfile(f, os.path.join(os.path.dirname(OUT), "onnx", os.path.basename(f)))
out["onnx_layernorm"] = lnm

with open(OUT, "w") as f:
    json.dump(out, f, indent=0, separators=(",", ":"))
print("wrote", OUT, os.path.getsize(OUT), "bytes")
for k, v in out.items():
    if isinstance(v, list):
        print(" ", k, len(v), "cases")
