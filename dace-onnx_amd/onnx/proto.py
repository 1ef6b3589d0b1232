"""A self-contained reader/writer for the part of the ONNX file format the
importer needs.

The reference takes an ``onnx.ModelProto`` (``daceml/onnx/onnx_importer.py:94-131``)
and walks ``graph.node / input / output / initializer / value_info`` and node
attributes (``:155-299``). The ``onnx`` package is not a dependency of this
build, so the same object model is provided here together with the protobuf
wire encoding of exactly those messages (field numbers from onnx.proto, IR
version 7): files written by ``save`` load in ``onnx``, and ``.onnx`` files
exported elsewhere load with ``load`` as long as they only use these fields.

``helper`` / ``numpy_helper`` / ``TensorProto`` mirror the names of the
``onnx`` package so graph-building code reads the same.
"""
import struct
import typing

import numpy as np

# ----------------------------------------------------------------------------- object model


class TensorProto:
    # element types (onnx.TensorProto.DataType)
    UNDEFINED, FLOAT, UINT8, INT8, UINT16, INT16, INT32, INT64, STRING, BOOL, FLOAT16, DOUBLE = range(12)

    def __init__(self, name="", dims=(), data_type=FLOAT, array: typing.Optional[np.ndarray] = None):
        self.name = name
        self.dims = list(dims)
        self.data_type = data_type
        self.array = array  # decoded contents


_NP_OF = {
    TensorProto.FLOAT: np.float32, TensorProto.UINT8: np.uint8, TensorProto.INT8: np.int8,
    TensorProto.UINT16: np.uint16, TensorProto.INT16: np.int16, TensorProto.INT32: np.int32,
    TensorProto.INT64: np.int64, TensorProto.BOOL: np.bool_, TensorProto.FLOAT16: np.float16,
    TensorProto.DOUBLE: np.float64,
}
_ONNX_OF = {np.dtype(v): k for k, v in _NP_OF.items()}


def tensor_dtype_to_np_dtype(data_type: int):
    return np.dtype(_NP_OF[data_type])


def np_dtype_to_tensor_dtype(dtype) -> int:
    return _ONNX_OF[np.dtype(dtype)]


class AttributeProto:
    UNDEFINED, FLOAT, INT, STRING, TENSOR, GRAPH, FLOATS, INTS, STRINGS = range(9)

    def __init__(self, name, value, type_=None):
        self.name = name
        self.value = value
        self.type = type_ if type_ is not None else self._infer_type(value)

    @staticmethod
    def _infer_type(v):
        if isinstance(v, bool) or isinstance(v, (int, np.integer)):
            return AttributeProto.INT
        if isinstance(v, (float, np.floating)):
            return AttributeProto.FLOAT
        if isinstance(v, (str, bytes)):
            return AttributeProto.STRING
        if isinstance(v, TensorProto):
            return AttributeProto.TENSOR
        if isinstance(v, (list, tuple)):
            if len(v) == 0 or all(isinstance(x, (int, np.integer)) for x in v):
                return AttributeProto.INTS
            if all(isinstance(x, (int, float, np.integer, np.floating)) for x in v):
                return AttributeProto.FLOATS
            if all(isinstance(x, (str, bytes)) for x in v):
                return AttributeProto.STRINGS
        raise TypeError(f"unsupported attribute value {v!r}")


class NodeProto:
    def __init__(self, op_type, inputs, outputs, name="", attributes=(), domain=""):
        self.op_type = op_type
        self.input = list(inputs)
        self.output = list(outputs)
        self.name = name
        self.attribute = list(attributes)
        self.domain = domain


class ValueInfoProto:
    def __init__(self, name, elem_type=TensorProto.FLOAT, shape=None):
        self.name = name
        self.elem_type = elem_type
        self.shape = None if shape is None else list(shape)  # ints, or str for symbolic dims


class GraphProto:
    def __init__(self, name="", nodes=(), inputs=(), outputs=(), initializers=(), value_info=()):
        self.name = name
        self.node = list(nodes)
        self.input = list(inputs)
        self.output = list(outputs)
        self.initializer = list(initializers)
        self.value_info = list(value_info)


class OperatorSetIdProto:
    def __init__(self, domain="", version=12):
        self.domain, self.version = domain, version


class ModelProto:
    def __init__(self, graph: GraphProto, ir_version=7, opset_imports=None, producer_name="dace_onnx_amd"):
        self.graph = graph
        self.ir_version = ir_version
        self.opset_import = list(opset_imports) if opset_imports is not None else [OperatorSetIdProto("", 12)]
        self.producer_name = producer_name


class helper:
    """``onnx.helper`` look-alikes."""

    @staticmethod
    def make_node(op_type, inputs, outputs, name="", domain="", **attributes) -> NodeProto:
        attrs = [AttributeProto(k, v) for k, v in attributes.items() if v is not None]
        return NodeProto(op_type, inputs, outputs, name, attrs, domain)

    @staticmethod
    def make_tensor_value_info(name, elem_type, shape) -> ValueInfoProto:
        return ValueInfoProto(name, elem_type, shape)

    @staticmethod
    def make_graph(nodes, name, inputs, outputs, initializer=(), value_info=()) -> GraphProto:
        return GraphProto(name, nodes, inputs, outputs, initializer, value_info)

    @staticmethod
    def make_model(graph, opset_imports=None, **kwargs) -> ModelProto:
        return ModelProto(graph, opset_imports=opset_imports, **kwargs)

    @staticmethod
    def make_opsetid(domain, version) -> OperatorSetIdProto:
        return OperatorSetIdProto(domain, version)

    @staticmethod
    def get_attribute_value(attr: AttributeProto):
        return attr.value


class numpy_helper:
    @staticmethod
    def from_array(arr: np.ndarray, name="") -> TensorProto:
        arr = np.asarray(arr)
        return TensorProto(name, arr.shape, np_dtype_to_tensor_dtype(arr.dtype), np.ascontiguousarray(arr))

    @staticmethod
    def to_array(t: TensorProto) -> np.ndarray:
        return t.array


# ----------------------------------------------------------------------------- wire format

_VARINT, _FIXED64, _BYTES, _FIXED32 = 0, 1, 2, 5


def _enc_varint(v: int) -> bytes:
    if v < 0:
        v += 1 << 64
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _key(field, wt) -> bytes:
    return _enc_varint((field << 3) | wt)


def _f_varint(field, v) -> bytes:
    return _key(field, _VARINT) + _enc_varint(int(v))


def _f_bytes(field, b) -> bytes:
    if isinstance(b, str):
        b = b.encode("utf-8")
    return _key(field, _BYTES) + _enc_varint(len(b)) + bytes(b)


def _f_float(field, v) -> bytes:
    return _key(field, _FIXED32) + struct.pack("<f", float(v))


def _ser_tensor(t: TensorProto) -> bytes:
    out = b"".join(_f_varint(1, d) for d in t.dims)
    out += _f_varint(2, t.data_type)
    if t.name:
        out += _f_bytes(8, t.name)
    arr = np.ascontiguousarray(t.array).astype(tensor_dtype_to_np_dtype(t.data_type), copy=False)
    out += _f_bytes(9, arr.astype(arr.dtype.newbyteorder("<"), copy=False).tobytes())
    return out


def _ser_attribute(a: AttributeProto) -> bytes:
    out = _f_bytes(1, a.name)
    A = AttributeProto
    if a.type == A.FLOAT:
        out += _f_float(2, a.value)
    elif a.type == A.INT:
        out += _f_varint(3, a.value)
    elif a.type == A.STRING:
        out += _f_bytes(4, a.value)
    elif a.type == A.TENSOR:
        out += _f_bytes(5, _ser_tensor(a.value))
    elif a.type == A.FLOATS:
        out += b"".join(_f_float(7, v) for v in a.value)
    elif a.type == A.INTS:
        out += b"".join(_f_varint(8, v) for v in a.value)
    elif a.type == A.STRINGS:
        out += b"".join(_f_bytes(9, v) for v in a.value)
    else:
        raise TypeError(f"attribute '{a.name}': type {a.type} cannot be written")
    out += _f_varint(20, a.type)
    return out


def _ser_node(n: NodeProto) -> bytes:
    out = b"".join(_f_bytes(1, i) for i in n.input)
    out += b"".join(_f_bytes(2, o) for o in n.output)
    if n.name:
        out += _f_bytes(3, n.name)
    out += _f_bytes(4, n.op_type)
    out += b"".join(_f_bytes(5, _ser_attribute(a)) for a in n.attribute)
    if n.domain:
        out += _f_bytes(7, n.domain)
    return out


def _ser_value_info(v: ValueInfoProto) -> bytes:
    tensor_type = _f_varint(1, v.elem_type)
    if v.shape is not None:
        dims = b""
        for d in v.shape:
            dim = _f_bytes(2, d) if isinstance(d, str) else _f_varint(1, d)
            dims += _f_bytes(1, dim)
        tensor_type += _f_bytes(2, dims)
    return _f_bytes(1, v.name) + _f_bytes(2, _f_bytes(1, tensor_type))


def _ser_graph(g: GraphProto) -> bytes:
    out = b"".join(_f_bytes(1, _ser_node(n)) for n in g.node)
    out += _f_bytes(2, g.name)
    out += b"".join(_f_bytes(5, _ser_tensor(t)) for t in g.initializer)
    out += b"".join(_f_bytes(11, _ser_value_info(v)) for v in g.input)
    out += b"".join(_f_bytes(12, _ser_value_info(v)) for v in g.output)
    out += b"".join(_f_bytes(13, _ser_value_info(v)) for v in g.value_info)
    return out


def serialize_model(m: ModelProto) -> bytes:
    out = _f_varint(1, m.ir_version)
    out += _f_bytes(2, m.producer_name)
    out += _f_bytes(7, _ser_graph(m.graph))
    for o in m.opset_import:
        out += _f_bytes(8, (_f_bytes(1, o.domain) if o.domain else b"") + _f_varint(2, o.version))
    return out


class _Reader:
    def __init__(self, buf: bytes):
        self.buf, self.pos = memoryview(buf), 0

    def done(self):
        return self.pos >= len(self.buf)

    def varint(self) -> int:
        shift = v = 0
        while True:
            if self.pos >= len(self.buf):
                raise ValueError("truncated varint")
            b = self.buf[self.pos]
            self.pos += 1
            v |= (b & 0x7F) << shift
            if not b & 0x80:
                return v
            shift += 7
            if shift > 70:
                raise ValueError("varint too long")

    def field(self):
        key = self.varint()
        field, wt = key >> 3, key & 7
        if wt == _VARINT:
            return field, wt, self.varint()
        if wt == _FIXED64:
            v = bytes(self.buf[self.pos:self.pos + 8])
            self.pos += 8
        elif wt == _BYTES:
            n = self.varint()
            v = bytes(self.buf[self.pos:self.pos + n])
            if len(v) != n:
                raise ValueError("truncated length-delimited field")
            self.pos += n
        elif wt == _FIXED32:
            v = bytes(self.buf[self.pos:self.pos + 4])
            self.pos += 4
        else:
            raise ValueError(f"unsupported wire type {wt}")
        return field, wt, v


def _signed(v: int) -> int:
    return v - (1 << 64) if v >= (1 << 63) else v


def _packed_varints(b: bytes):
    r, out = _Reader(b), []
    while not r.done():
        out.append(_signed(r.varint()))
    return out


def _parse_tensor(b: bytes) -> TensorProto:
    t = TensorProto()
    raw = None
    typed: typing.Dict[int, list] = {4: [], 5: [], 7: [], 10: [], 11: []}
    r = _Reader(b)
    while not r.done():
        f, wt, v = r.field()
        if f == 1:
            t.dims.extend(_packed_varints(v) if wt == _BYTES else [_signed(v)])
        elif f == 2:
            t.data_type = v
        elif f == 8:
            t.name = v.decode("utf-8")
        elif f == 9:
            raw = v
        elif f == 4:
            typed[4].extend(struct.unpack(f"<{len(v) // 4}f", v) if wt == _BYTES else struct.unpack("<f", v))
        elif f == 10:
            typed[10].extend(struct.unpack(f"<{len(v) // 8}d", v) if wt == _BYTES else struct.unpack("<d", v))
        elif f in (5, 7, 11):
            typed[f].extend(_packed_varints(v) if wt == _BYTES else [_signed(v)])
    dtype = tensor_dtype_to_np_dtype(t.data_type)
    if raw is not None:
        arr = np.frombuffer(raw, dtype=dtype.newbyteorder("<")).astype(dtype)
    else:
        src = {TensorProto.FLOAT: 4, TensorProto.DOUBLE: 10, TensorProto.INT64: 7}.get(t.data_type, 5)
        arr = np.array(typed[src]).astype(dtype)
    t.array = arr.reshape(t.dims)
    return t


def _parse_attribute(b: bytes) -> AttributeProto:
    name, typ = "", None
    f_, i_, s_, t_ = None, None, None, None
    floats, ints, strings = [], [], []
    r = _Reader(b)
    while not r.done():
        f, wt, v = r.field()
        if f == 1:
            name = v.decode("utf-8")
        elif f == 2:
            f_ = struct.unpack("<f", v)[0]
        elif f == 3:
            i_ = _signed(v)
        elif f == 4:
            s_ = v
        elif f == 5:
            t_ = _parse_tensor(v)
        elif f == 7:
            floats.extend(struct.unpack(f"<{len(v) // 4}f", v) if wt == _BYTES else struct.unpack("<f", v))
        elif f == 8:
            ints.extend(_packed_varints(v) if wt == _BYTES else [_signed(v)])
        elif f == 9:
            strings.append(v)
        elif f == 20:
            typ = v
    A = AttributeProto
    if typ is None:  # IR < 3 files carry no type tag
        typ = (A.FLOAT if f_ is not None else A.INT if i_ is not None else A.STRING if s_ is not None else
               A.TENSOR if t_ is not None else A.FLOATS if floats else A.INTS if ints else A.STRINGS)
    value = {A.FLOAT: f_, A.INT: i_, A.STRING: s_.decode("utf-8") if s_ is not None else None, A.TENSOR: t_,
             A.FLOATS: list(floats), A.INTS: list(ints),
             A.STRINGS: [x.decode("utf-8") for x in strings]}.get(typ)
    if typ not in (A.FLOAT, A.INT, A.STRING, A.TENSOR, A.FLOATS, A.INTS, A.STRINGS):
        raise ValueError(f"attribute '{name}': type {typ} is not supported")
    if typ == A.FLOAT and value is None:
        value = 0.0
    if typ == A.INT and value is None:
        value = 0
    return AttributeProto(name, value, typ)


def _parse_node(b: bytes) -> NodeProto:
    n = NodeProto("", [], [])
    r = _Reader(b)
    while not r.done():
        f, _, v = r.field()
        if f == 1:
            n.input.append(v.decode("utf-8"))
        elif f == 2:
            n.output.append(v.decode("utf-8"))
        elif f == 3:
            n.name = v.decode("utf-8")
        elif f == 4:
            n.op_type = v.decode("utf-8")
        elif f == 5:
            n.attribute.append(_parse_attribute(v))
        elif f == 7:
            n.domain = v.decode("utf-8")
    return n


def _parse_value_info(b: bytes) -> ValueInfoProto:
    vi = ValueInfoProto("", TensorProto.UNDEFINED, None)
    r = _Reader(b)
    while not r.done():
        f, _, v = r.field()
        if f == 1:
            vi.name = v.decode("utf-8")
        elif f == 2:  # TypeProto
            rt = _Reader(v)
            while not rt.done():
                ft, _, vt = rt.field()
                if ft != 1:  # only tensor_type
                    continue
                rtt = _Reader(vt)
                while not rtt.done():
                    f2, _, v2 = rtt.field()
                    if f2 == 1:
                        vi.elem_type = v2
                    elif f2 == 2:
                        vi.shape = []
                        rs = _Reader(v2)
                        while not rs.done():
                            f3, _, v3 = rs.field()
                            if f3 != 1:
                                continue
                            dim = None
                            rd = _Reader(v3)
                            while not rd.done():
                                f4, _, v4 = rd.field()
                                if f4 == 1:
                                    dim = _signed(v4)
                                elif f4 == 2:
                                    dim = v4.decode("utf-8")
                            vi.shape.append(dim if dim is not None else "?")
    return vi


def _parse_graph(b: bytes) -> GraphProto:
    g = GraphProto()
    r = _Reader(b)
    while not r.done():
        f, _, v = r.field()
        if f == 1:
            g.node.append(_parse_node(v))
        elif f == 2:
            g.name = v.decode("utf-8")
        elif f == 5:
            g.initializer.append(_parse_tensor(v))
        elif f == 11:
            g.input.append(_parse_value_info(v))
        elif f == 12:
            g.output.append(_parse_value_info(v))
        elif f == 13:
            g.value_info.append(_parse_value_info(v))
    return g


def parse_model(b: bytes) -> ModelProto:
    graph, ir, opsets, producer = None, 7, [], ""
    r = _Reader(b)
    while not r.done():
        f, _, v = r.field()
        if f == 1:
            ir = v
        elif f == 2:
            producer = v.decode("utf-8")
        elif f == 7:
            graph = _parse_graph(v)
        elif f == 8:
            o = OperatorSetIdProto("", 0)
            ro = _Reader(v)
            while not ro.done():
                fo, _, vo = ro.field()
                if fo == 1:
                    o.domain = vo.decode("utf-8")
                elif fo == 2:
                    o.version = vo
            opsets.append(o)
    if graph is None:
        raise ValueError("not an ONNX ModelProto: no graph field")
    return ModelProto(graph, ir, opsets, producer)


def load(path_or_bytes) -> ModelProto:
    """``onnx.load``: read a ``.onnx`` file (or parse serialized bytes)."""
    if isinstance(path_or_bytes, (bytes, bytearray, memoryview)):
        return parse_model(bytes(path_or_bytes))
    with open(path_or_bytes, "rb") as f:
        return parse_model(f.read())


def save(model: ModelProto, path) -> None:
    """``onnx.save``."""
    with open(path, "wb") as f:
        f.write(serialize_model(model))
