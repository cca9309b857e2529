"""A minimal ONNX reader for the tests: protobuf wire format decoded by hand (no onnx package here).
Returns plain dicts: graph inputs with shapes, initializers as numpy arrays, nodes with attributes."""
import struct

import numpy as np


def _varint(buf, pos):
    result, shift = 0, 0
    while True:
        b = buf[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7


def _fields(buf):
    """Yields (field_number, wire_type, value) for one message."""
    pos, n = 0, len(buf)
    while pos < n:
        key, pos = _varint(buf, pos)
        fno, wt = key >> 3, key & 7
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
        yield fno, wt, val


def _signed(v):
    return v - (1 << 64) if v >= (1 << 63) else v


def _packed_varints(buf):
    out, pos = [], 0
    while pos < len(buf):
        v, pos = _varint(buf, pos)
        out.append(_signed(v))
    return out


_DTYPES = {1: np.float32, 2: np.uint8, 3: np.int8, 6: np.int32, 7: np.int64, 9: np.bool_, 11: np.float64}


def _tensor(buf):
    dims, dtype, name, raw = [], 1, "", None
    floats, int32s, int64s = [], [], []
    for fno, wt, val in _fields(buf):
        if fno == 1:
            dims += _packed_varints(val) if wt == 2 else [_signed(val)]
        elif fno == 2:
            dtype = val
        elif fno == 4:
            floats += list(struct.unpack("<%df" % (len(val) // 4), val)) if wt == 2 else [struct.unpack("<f", val)[0]]
        elif fno == 5:
            int32s += _packed_varints(val) if wt == 2 else [_signed(val)]
        elif fno == 7:
            int64s += _packed_varints(val) if wt == 2 else [_signed(val)]
        elif fno == 8:
            name = bytes(val).decode()
        elif fno == 9:
            raw = bytes(val)
    np_dt = _DTYPES.get(dtype)
    if np_dt is None:
        raise ValueError("tensor %s: unsupported data type %d" % (name, dtype))
    if raw is not None:
        arr = np.frombuffer(raw, dtype=np_dt).copy()
    elif floats:
        arr = np.array(floats, dtype=np_dt)
    elif int64s:
        arr = np.array(int64s, dtype=np_dt)
    else:
        arr = np.array(int32s, dtype=np_dt)
    return name, arr.reshape(dims)


def _attribute(buf):
    name, out = "", {}
    ints, floats = [], []
    for fno, wt, val in _fields(buf):
        if fno == 1:
            name = bytes(val).decode()
        elif fno == 2:
            out["f"] = struct.unpack("<f", val)[0]
        elif fno == 3:
            out["i"] = _signed(val)
        elif fno == 4:
            out["s"] = bytes(val).decode()
        elif fno == 5:
            out["t"] = _tensor(val)[1]
        elif fno == 7:
            floats += list(struct.unpack("<%df" % (len(val) // 4), val)) if wt == 2 else [struct.unpack("<f", val)[0]]
        elif fno == 8:
            ints += _packed_varints(val) if wt == 2 else [_signed(val)]
    if ints:
        return name, ints
    if floats:
        return name, floats
    for k in ("i", "f", "s", "t"):
        if k in out:
            return name, out[k]
    return name, None


def _node(buf):
    n = {"inputs": [], "outputs": [], "name": "", "op": "", "attrs": {}}
    for fno, wt, val in _fields(buf):
        if fno == 1:
            n["inputs"].append(bytes(val).decode())
        elif fno == 2:
            n["outputs"].append(bytes(val).decode())
        elif fno == 3:
            n["name"] = bytes(val).decode()
        elif fno == 4:
            n["op"] = bytes(val).decode()
        elif fno == 5:
            k, v = _attribute(val)
            n["attrs"][k] = v
    return n


def _value_info(buf):
    name, shape = "", []
    for fno, wt, val in _fields(buf):
        if fno == 1:
            name = bytes(val).decode()
        elif fno == 2:  # TypeProto
            for f2, _, v2 in _fields(val):
                if f2 == 1:  # tensor_type
                    for f3, _, v3 in _fields(v2):
                        if f3 == 2:  # shape
                            for f4, _, v4 in _fields(v3):
                                if f4 == 1:  # dim
                                    d = None
                                    for f5, _, v5 in _fields(v4):
                                        if f5 == 1:
                                            d = _signed(v5)
                                        elif f5 == 2:
                                            d = bytes(v5).decode()
                                    shape.append(d)
    return name, shape


def load(path):
    with open(path, "rb") as f:
        buf = memoryview(f.read())
    graph = None
    for fno, wt, val in _fields(buf):
        if fno == 7:
            graph = val
    if graph is None:
        raise ValueError("%s: no graph" % path)
    g = {"nodes": [], "initializers": {}, "inputs": [], "outputs": []}
    for fno, wt, val in _fields(graph):
        if fno == 1:
            g["nodes"].append(_node(val))
        elif fno == 5:
            name, arr = _tensor(val)
            g["initializers"][name] = arr
        elif fno == 11:
            g["inputs"].append(_value_info(val))
        elif fno == 12:
            g["outputs"].append(_value_info(val))
    g["inputs"] = [(n, s) for n, s in g["inputs"] if n not in g["initializers"]]
    return g
