"""A protobuf encoder for ONNX models, written from the field numbers of onnx.proto
(crates/core/src/onnx/onnx.proto in the reference: ModelProto 340-412, GraphProto 439-470,
NodeProto 196-213, AttributeProto 114-177, TensorProto 479-616, ValueInfoProto 179-187,
TypeProto 665-738, TensorShapeProto 646-661, OperatorSetIdProto 744-754).

Test infrastructure only: it produces the bytes the loader under test must read, the way the
`onnx` Python package (not installed here) would.  Nothing in the product imports it."""
import struct

import numpy as np

FLOAT, INT32, INT64, BOOL, FLOAT16, DOUBLE = 1, 6, 7, 9, 10, 11
_DT = {np.dtype(np.float32): FLOAT, np.dtype(np.int32): INT32, np.dtype(np.int64): INT64, np.dtype(np.bool_): BOOL,
       np.dtype(np.float16): FLOAT16, np.dtype(np.float64): DOUBLE}
A_FLOAT, A_INT, A_STRING, A_TENSOR, A_GRAPH, A_FLOATS, A_INTS = 1, 2, 3, 4, 5, 6, 7


def varint(v):
    v &= (1 << 64) - 1  # negative int64 -> ten-byte two's complement
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def key(field, wire):
    return varint((field << 3) | wire)


def f_varint(field, v):
    return key(field, 0) + varint(int(v))


def f_bytes(field, b):
    if isinstance(b, str):
        b = b.encode()
    return key(field, 2) + varint(len(b)) + bytes(b)


def f_float(field, v):
    return key(field, 5) + struct.pack("<f", v)


def packed_varints(field, vals):
    return f_bytes(field, b"".join(varint(int(v)) for v in vals))


def unpacked_varints(field, vals):
    return b"".join(f_varint(field, v) for v in vals)


def tensor(name, array, raw=True, packed=True):
    """TensorProto.  raw=False stores float_data / int32_data / int64_data instead of raw_data."""
    a = np.asarray(array)
    rep = packed_varints if packed else unpacked_varints
    out = rep(1, a.shape) if a.ndim else b""
    out += f_varint(2, _DT[a.dtype])
    if raw:
        out += f_bytes(9, a.astype(a.dtype.newbyteorder("<")).tobytes())
    elif a.dtype == np.float32:
        flat = a.ravel()
        out += f_bytes(4, flat.astype("<f4").tobytes()) if packed else b"".join(f_float(4, float(v)) for v in flat)
    elif a.dtype == np.int32:
        out += rep(5, a.ravel())
    elif a.dtype == np.int64:
        out += rep(7, a.ravel())
    else:
        raise ValueError("typed storage exists for float32, int32 and int64 only")
    if name is not None:
        out += f_bytes(8, name)
    return out


def attribute(name, value, with_type=True, omit_zero=False):
    """AttributeProto for a Python value: int, float, str, list of ints/floats, numpy array (tensor),
    or ('graph', bytes).  omit_zero leaves out a zero-valued scalar payload (the type tag still says what it is)."""
    out = f_bytes(1, name)
    if isinstance(value, tuple) and value[0] == "graph":
        body, ty = f_bytes(6, value[1]), A_GRAPH
    elif isinstance(value, bool) or isinstance(value, (int, np.integer)):
        body, ty = (b"" if omit_zero and int(value) == 0 else f_varint(3, int(value))), A_INT
    elif isinstance(value, (float, np.floating)):
        body, ty = (b"" if omit_zero and float(value) == 0.0 else f_float(2, float(value))), A_FLOAT
    elif isinstance(value, str):
        body, ty = f_bytes(4, value), A_STRING
    elif isinstance(value, np.ndarray):
        body, ty = f_bytes(5, tensor(None, value)), A_TENSOR
    elif isinstance(value, (list, tuple)) and all(isinstance(v, (float, np.floating)) for v in value) and value:
        body, ty = f_bytes(7, b"".join(struct.pack("<f", v) for v in value)), A_FLOATS
    elif isinstance(value, (list, tuple)):
        body, ty = unpacked_varints(8, value), A_INTS   # proto2 writers emit repeated int64 unpacked
    else:
        raise TypeError(value)
    out += body
    if with_type:
        out += f_varint(20, ty)
    return out


def node(op_type, inputs, outputs, name="", domain=None, attr_opts=None, **attrs):
    out = b"".join(f_bytes(1, i) for i in inputs) + b"".join(f_bytes(2, o) for o in outputs)
    if name:
        out += f_bytes(3, name)
    out += f_bytes(4, op_type)
    for k, v in attrs.items():
        out += f_bytes(5, attribute(k, v, **(attr_opts or {})))
    if domain is not None:
        out += f_bytes(7, domain)
    return out


def value_info(name, elem_type=FLOAT, dims=(), with_type=True, with_shape=True, kind="tensor"):
    """dims: ints (dim_value) or strings (dim_param).  kind='sequence' makes a non-tensor type."""
    out = f_bytes(1, name)
    if not with_type:
        return out
    if kind == "sequence":
        return out + f_bytes(2, f_bytes(4, b""))
    shape = b""
    for d in dims:
        shape += f_bytes(1, f_bytes(2, d) if isinstance(d, str) else f_varint(1, d))
    t = f_varint(1, elem_type)
    if with_shape:
        t += f_bytes(2, shape)
    return out + f_bytes(2, f_bytes(1, t))


def graph(nodes, initializers=(), inputs=(), outputs=(), name="g"):
    out = b"".join(f_bytes(1, n) for n in nodes)
    out += f_bytes(2, name)
    out += b"".join(f_bytes(5, t) for t in initializers)
    out += b"".join(f_bytes(11, v) for v in inputs)
    out += b"".join(f_bytes(12, v) for v in outputs)
    return out


def model(graph_bytes, opsets=(("", 13),), ir_version=8, producer="altius_amd tests"):
    out = f_varint(1, ir_version) + f_bytes(2, producer)
    if graph_bytes is not None:
        out += f_bytes(7, graph_bytes)
    for domain, version in opsets:
        out += f_bytes(8, (f_bytes(1, domain) if domain is not None else b"") + f_varint(2, version))
    return out
