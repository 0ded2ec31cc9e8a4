"""Minimal protobuf wire-format reader for ONNX files (no protobuf/onnx packages).

Only the fields needed to read the Gemm / Conv / MaxPool fixtures are decoded.
Field numbers follow the ONNX schema (ModelProto.graph = 7, GraphProto.node = 1,
initializer = 5, input = 11, output = 12, NodeProto input/output/name/op_type/attribute
= 1..5, AttributeProto name/f/i/s/t/floats/ints = 1,2,3,4,5,7,8, TensorProto dims = 1,
data_type = 2, float_data = 4, int32_data = 5, int64_data = 7, name = 8, raw_data = 9).
"""
import struct

import numpy as np

_DTYPES = {1: np.float32, 2: np.uint8, 3: np.int8, 6: np.int32, 7: np.int64, 11: np.float64}


def _varint(buf, pos):
    result = shift = 0
    while True:
        b = buf[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7


def _fields(buf):
    """Yield (field_number, wire_type, value) for one message."""
    pos, end = 0, len(buf)
    while pos < end:
        key, pos = _varint(buf, pos)
        num, wt = key >> 3, key & 7
        if wt == 0:
            val, pos = _varint(buf, pos)
        elif wt == 1:
            val = buf[pos:pos + 8]
            pos += 8
        elif wt == 2:
            ln, pos = _varint(buf, pos)
            val = buf[pos:pos + ln]
            pos += ln
        elif wt == 5:
            val = buf[pos:pos + 4]
            pos += 4
        else:
            raise ValueError("unsupported wire type %d" % wt)
        yield num, wt, val


def _signed(v):
    return v - (1 << 64) if v >= (1 << 63) else v


def _ints(wt, val):
    if wt == 0:
        return [_signed(val)]
    out, pos = [], 0
    while pos < len(val):
        v, pos = _varint(val, pos)
        out.append(_signed(v))
    return out


def _tensor(buf):
    dims, dtype, name, raw = [], 1, "", None
    floats, i32, i64 = [], [], []
    for num, wt, val in _fields(buf):
        if num == 1:
            dims += _ints(wt, val)
        elif num == 2:
            dtype = val
        elif num == 4:
            floats += list(struct.unpack("<%df" % (len(val) // 4), val)) if wt == 2 else \
                [struct.unpack("<f", val)[0]]
        elif num == 5:
            i32 += _ints(wt, val)
        elif num == 7:
            i64 += _ints(wt, val)
        elif num == 8:
            name = bytes(val).decode()
        elif num == 9:
            raw = bytes(val)
    np_dtype = _DTYPES[dtype]
    if raw is not None:
        arr = np.frombuffer(raw, dtype=np.dtype(np_dtype).newbyteorder("<")).astype(np_dtype)
    elif floats:
        arr = np.array(floats, np_dtype)
    elif i64:
        arr = np.array(i64, np_dtype)
    else:
        arr = np.array(i32, np_dtype)
    return name, arr.reshape(dims)


def _attribute(buf):
    name, value, floats, ints = "", None, [], []
    for num, wt, val in _fields(buf):
        if num == 1:
            name = bytes(val).decode()
        elif num == 2:
            value = struct.unpack("<f", val)[0]
        elif num == 3:
            value = _signed(val)
        elif num == 4:
            value = bytes(val).decode()
        elif num == 5:
            value = _tensor(val)[1]
        elif num == 7:
            floats += list(struct.unpack("<%df" % (len(val) // 4), val)) if wt == 2 else \
                [struct.unpack("<f", val)[0]]
        elif num == 8:
            ints += _ints(wt, val)
    if value is None:
        value = ints if ints else floats
    return name, value


def _node(buf):
    node = {"inputs": [], "outputs": [], "name": "", "op_type": "", "attrs": {}}
    for num, _, val in _fields(buf):
        if num == 1:
            node["inputs"].append(bytes(val).decode())
        elif num == 2:
            node["outputs"].append(bytes(val).decode())
        elif num == 3:
            node["name"] = bytes(val).decode()
        elif num == 4:
            node["op_type"] = bytes(val).decode()
        elif num == 5:
            k, v = _attribute(val)
            node["attrs"][k] = v
    return node


def _value_info(buf):
    name, shape, elem = "", [], 0
    for num, _, val in _fields(buf):
        if num == 1:
            name = bytes(val).decode()
        elif num == 2:                                   # TypeProto
            for n2, _, v2 in _fields(val):
                if n2 == 1:                              # tensor_type
                    for n3, _, v3 in _fields(v2):
                        if n3 == 1:
                            elem = v3
                        elif n3 == 2:                    # TensorShapeProto
                            for n4, _, v4 in _fields(v3):
                                if n4 == 1:              # Dimension
                                    d = None
                                    for n5, _, v5 in _fields(v4):
                                        if n5 == 1:
                                            d = _signed(v5)
                                        elif n5 == 2:
                                            d = bytes(v5).decode()
                                    shape.append(d)
    return name, elem, shape


def load(path):
    """Return {'nodes': [...], 'initializers': {name: ndarray}, 'inputs': [(name, elem, shape)],
    'outputs': [...]} for an ONNX file."""
    with open(path, "rb") as f:
        buf = memoryview(f.read())
    graph = None
    for num, _, val in _fields(buf):
        if num == 7:
            graph = val
    if graph is None:
        raise ValueError("no graph in " + path)
    out = {"nodes": [], "initializers": {}, "inputs": [], "outputs": []}
    for num, _, val in _fields(graph):
        if num == 1:
            out["nodes"].append(_node(val))
        elif num == 5:
            name, arr = _tensor(val)
            out["initializers"][name] = arr
        elif num == 11:
            out["inputs"].append(_value_info(val))
        elif num == 12:
            out["outputs"].append(_value_info(val))
    out["inputs"] = [i for i in out["inputs"] if i[0] not in out["initializers"]]
    return out
