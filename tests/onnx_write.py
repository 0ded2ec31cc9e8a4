"""Minimal ONNX (protobuf wire format) writer for tests: just enough of ModelProto / GraphProto / NodeProto /
TensorProto / ValueInfoProto to build small graphs that the C++ front end then parses."""
import struct

import numpy as np

_ONNX_TYPE = {np.dtype(np.float32): 1, np.dtype(np.uint8): 2, np.dtype(np.int8): 3, np.dtype(np.int32): 6,
              np.dtype(np.int64): 7}


def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _key(num, wire):
    return _varint((num << 3) | wire)


def _bytes(num, payload):
    return _key(num, 2) + _varint(len(payload)) + payload


def _int(num, v):
    return _key(num, 0) + _varint(v)


def tensor(name, arr):
    arr = np.ascontiguousarray(arr)
    msg = b"".join(_int(1, d) for d in arr.shape) + _int(2, _ONNX_TYPE[arr.dtype]) + _bytes(8, name.encode())
    return msg + _bytes(9, arr.astype(arr.dtype.newbyteorder("<")).tobytes())


def attribute(name, value):
    msg = _bytes(1, name.encode())
    if isinstance(value, float):
        return msg + _key(2, 5) + struct.pack("<f", value) + _int(20, 1)
    if isinstance(value, int):
        return msg + _int(3, value) + _int(20, 2)
    if isinstance(value, str):
        return msg + _bytes(4, value.encode()) + _int(20, 3)
    return msg + b"".join(_int(8, int(v)) for v in value) + _int(20, 7)      # ints


def node(op_type, inputs, outputs, name="", **attrs):
    msg = b"".join(_bytes(1, i.encode()) for i in inputs) + b"".join(_bytes(2, o.encode()) for o in outputs)
    msg += _bytes(3, name.encode()) + _bytes(4, op_type.encode())
    return msg + b"".join(_bytes(5, attribute(k, v)) for k, v in attrs.items())


def value_info(name, elem_type, shape):
    # an int is a dim_value, a string a dim_param (a named, parametric dimension)
    dims = b"".join(_bytes(1, _bytes(2, d.encode()) if isinstance(d, str) else _int(1, d)) for d in shape)
    tensor_type = _int(1, elem_type) + _bytes(2, dims)
    return _bytes(1, name.encode()) + _bytes(2, _bytes(1, tensor_type))


def model(nodes, initializers, inputs, outputs, graph_name="g"):
    """nodes: list of node(); initializers: {name: ndarray}; inputs / outputs: [(name, elem_type, shape)]."""
    graph = b"".join(_bytes(1, n) for n in nodes) + _bytes(2, graph_name.encode())
    graph += b"".join(_bytes(5, tensor(k, v)) for k, v in initializers.items())
    graph += b"".join(_bytes(11, value_info(*i)) for i in inputs) + b"".join(_bytes(12, value_info(*o)) for o in outputs)
    return _int(1, 8) + _bytes(7, graph) + _bytes(8, _bytes(2, _int(2, 13)))   # ir_version, graph, opset 13
