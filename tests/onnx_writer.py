"""A minimal ONNX (protobuf wire format) writer for tests: enough of ModelProto / GraphProto /
NodeProto / TensorProto / ValueInfoProto to describe small quantized graphs without the onnx
package.  Field numbers are onnx.proto's."""
import struct

import numpy as np

FLOAT, UINT8, INT8, INT32, INT64, FLOAT16 = 1, 2, 3, 6, 7, 10
_NP2ONNX = {np.dtype(np.float32): FLOAT, np.dtype(np.uint8): UINT8, np.dtype(np.int8): INT8,
            np.dtype(np.int32): INT32, np.dtype(np.int64): INT64, np.dtype(np.float16): FLOAT16}


def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7f
        v >>= 7
        out.append(b | (0x80 if v else 0))
        if not v:
            return bytes(out)


def _key(field, wire_type):
    return _varint(field << 3 | wire_type)


def _bytes(field, payload):
    return _key(field, 2) + _varint(len(payload)) + payload


def _int(field, v):
    return _key(field, 0) + _varint(v)


def tensor(name, array):
    a = np.ascontiguousarray(array)
    out = b"".join(_int(1, d) for d in a.shape)
    out += _int(2, _NP2ONNX[a.dtype]) + _bytes(8, name.encode()) + _bytes(9, a.tobytes())
    return out


def attribute(name, value):
    out = _bytes(1, name.encode())
    if isinstance(value, int):
        return out + _int(3, value) + _int(20, 2)
    if isinstance(value, float):
        return out + _key(2, 5) + struct.pack("<f", value) + _int(20, 1)
    if isinstance(value, str):
        return out + _bytes(4, value.encode()) + _int(20, 3)
    if isinstance(value, (list, tuple)):
        return out + b"".join(_int(8, int(v)) for v in value) + _int(20, 7)
    raise TypeError(type(value))


def node(op_type, inputs, outputs, domain="", **attrs):
    out = b"".join(_bytes(1, i.encode()) for i in inputs)
    out += b"".join(_bytes(2, o.encode()) for o in outputs)
    out += _bytes(4, op_type.encode())
    out += b"".join(_bytes(5, attribute(k, v)) for k, v in attrs.items())
    if domain:
        out += _bytes(7, domain.encode())
    return out


def value_info(name, elem_type, dims):
    shape = b"".join(_bytes(1, _int(1, d)) for d in dims)
    tensor_type = _int(1, elem_type) + _bytes(2, shape)
    return _bytes(1, name.encode()) + _bytes(2, _bytes(1, tensor_type))


def model(nodes, inputs, outputs, initializers=()):
    """nodes: encoded nodes; inputs / outputs: (name, elem_type, dims); initializers: (name, array)."""
    g = b"".join(_bytes(1, n) for n in nodes) + _bytes(2, b"g")
    g += b"".join(_bytes(5, tensor(n, a)) for n, a in initializers)
    g += b"".join(_bytes(11, value_info(*i)) for i in inputs)
    g += b"".join(_bytes(12, value_info(*o)) for o in outputs)
    opset = _bytes(1, b"") + _int(2, 19)
    return _int(1, 8) + _bytes(8, opset) + _bytes(7, g)
