"""Writes ONNX files for the benchmark models and the tests (protobuf wire format by hand; the reference's tests do the same in
C++, tests/common/onnx_proto_helpers.h)."""
import struct

import numpy as np


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


def _key(fno, wt):
    return _varint((fno << 3) | wt)


def _ld(fno, payload):
    return _key(fno, 2) + _varint(len(payload)) + payload


def _vi(fno, v):
    return _key(fno, 0) + _varint(v)


_ONNX_TYPE = {np.dtype(np.float32): 1, np.dtype(np.uint8): 2, np.dtype(np.int8): 3, np.dtype(np.int32): 6, np.dtype(np.int64): 7}


def tensor(name, arr):
    arr = np.ascontiguousarray(arr)
    t = b"".join(_vi(1, d) for d in arr.shape)
    t += _vi(2, _ONNX_TYPE[arr.dtype]) + _ld(8, name.encode()) + _ld(9, arr.tobytes())
    return t


def attribute(name, value):
    a = _ld(1, name.encode())
    if isinstance(value, float):
        a += _key(2, 5) + struct.pack("<f", value) + _vi(20, 1)
    elif isinstance(value, int):
        a += _vi(3, value) + _vi(20, 2)
    elif isinstance(value, str):
        a += _ld(4, value.encode()) + _vi(20, 3)
    elif isinstance(value, np.ndarray):      # a tensor attribute (the value of a Constant node)
        a += _ld(5, tensor("", value)) + _vi(20, 4)
    else:
        a += b"".join(_vi(8, int(v)) for v in value) + _vi(20, 7)
    return a


def node(op, inputs, outputs, **attrs):
    n = b"".join(_ld(1, i.encode()) for i in inputs) + b"".join(_ld(2, o.encode()) for o in outputs)
    n += _ld(4, op.encode()) + b"".join(_ld(5, attribute(k, v)) for k, v in attrs.items())
    return n


def value_info(name, elem_type, shape):
    # an int is a dim_value, a str a dim_param (a named, run-time dimension)
    dims = b"".join(_ld(1, _ld(2, d.encode()) if isinstance(d, str) else _vi(1, d)) for d in shape)
    ttype = _vi(1, elem_type) + _ld(2, dims)
    return _ld(1, name.encode()) + _ld(2, _ld(1, ttype))


def model(nodes, inputs, outputs, initializers, name="g"):
    """inputs/outputs: [(name, numpy dtype, shape)], initializers: {name: array}"""
    g = b"".join(_ld(1, n) for n in nodes) + _ld(2, name.encode())
    g += b"".join(_ld(5, tensor(k, v)) for k, v in initializers.items())
    g += b"".join(_ld(11, value_info(n, _ONNX_TYPE[np.dtype(dt)], s)) for n, dt, s in inputs)
    g += b"".join(_ld(12, value_info(n, _ONNX_TYPE[np.dtype(dt)], s)) for n, dt, s in outputs)
    return _vi(1, 8) + _ld(8, _ld(2, _vi(2, 17))) + _ld(7, g)  # ir_version 8, opset 17


def write(path, *args, **kw):
    with open(path, "wb") as f:
        f.write(model(*args, **kw))
