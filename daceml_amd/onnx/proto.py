"""Reader for serialized ONNX models (protobuf wire format), without the ``onnx`` package.

Only what the importer needs is decoded: graph nodes with their attributes, initializers, graph inputs /
outputs / value infos with static shapes, and the default-domain opset version. Field numbers follow
onnx.proto3 (ModelProto.graph = 7, GraphProto.node = 1, NodeProto.attribute = 5, TensorProto.raw_data = 9, ...).
The decoded objects carry the same field names the ``onnx`` Python classes expose, which is what
daceml/onnx/onnx_importer.py:145-302 reads.
"""
import struct
from typing import Any, Dict, Iterator, List, Optional, Tuple

import numpy as np

# TensorProto.DataType -> numpy
TENSOR_DTYPES = {1: np.float32, 2: np.uint8, 3: np.int8, 4: np.uint16, 5: np.int16, 6: np.int32, 7: np.int64,
                 9: np.bool_, 10: np.float16, 11: np.float64, 12: np.uint32, 13: np.uint64}


class ProtoError(ValueError):
    pass


def _varint(buf: bytes, pos: int) -> Tuple[int, int]:
    result, shift = 0, 0
    while True:
        if pos >= len(buf):
            raise ProtoError("truncated varint")
        b = buf[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7
        if shift > 70:
            raise ProtoError("varint too long")


def _signed(v: int) -> int:
    return v - (1 << 64) if v >= 1 << 63 else v


def fields(buf: bytes) -> Iterator[Tuple[int, int, Any]]:
    """Yields (field number, wire type, value); value is an int for varint / fixed fields and a bytes slice for
    length-delimited ones."""
    pos, n = 0, len(buf)
    while pos < n:
        key, pos = _varint(buf, pos)
        num, wt = key >> 3, key & 7
        if wt == 0:
            v, pos = _varint(buf, pos)
        elif wt == 1:
            if pos + 8 > n:
                raise ProtoError("truncated fixed64")
            v = buf[pos:pos + 8]
            pos += 8
        elif wt == 2:
            ln, pos = _varint(buf, pos)
            if pos + ln > n:
                raise ProtoError("truncated length-delimited field %d" % num)
            v = buf[pos:pos + ln]
            pos += ln
        elif wt == 5:
            if pos + 4 > n:
                raise ProtoError("truncated fixed32")
            v = buf[pos:pos + 4]
            pos += 4
        else:
            raise ProtoError("unsupported wire type %d (field %d)" % (wt, num))
        yield num, wt, v


def _packed_varints(wt: int, v) -> List[int]:
    if wt == 0:
        return [_signed(v)]
    out, pos = [], 0
    while pos < len(v):
        x, pos = _varint(v, pos)
        out.append(_signed(x))
    return out


def _packed_fixed(wt: int, v, fmt: str, size: int) -> List:
    if wt in (1, 5):
        return [struct.unpack("<" + fmt, v)[0]]
    return list(struct.unpack("<%d%s" % (len(v) // size, fmt), v))


class TensorProto:
    def __init__(self, buf: bytes):
        self.dims: List[int] = []
        self.data_type = 0
        self.name = ""
        raw = None
        floats, int32s, int64s, doubles, uint64s = [], [], [], [], []
        for num, wt, v in fields(buf):
            if num == 1:
                self.dims += _packed_varints(wt, v)
            elif num == 2:
                self.data_type = v
            elif num == 4:
                floats += _packed_fixed(wt, v, "f", 4)
            elif num == 5:
                int32s += _packed_varints(wt, v)
            elif num == 7:
                int64s += _packed_varints(wt, v)
            elif num == 8:
                self.name = v.decode("utf-8")
            elif num == 9:
                raw = bytes(v)
            elif num == 10:
                doubles += _packed_fixed(wt, v, "d", 8)
            elif num == 11:
                uint64s += _packed_varints(wt, v)
            elif num in (13, 14) and (num == 13 or v == 1):
                raise ProtoError("tensor %r uses external data, which is not supported" % self.name)
        if self.data_type not in TENSOR_DTYPES:
            raise ProtoError("tensor %r has unsupported data type %d" % (self.name, self.data_type))
        dt = np.dtype(TENSOR_DTYPES[self.data_type])
        shape = tuple(self.dims)
        if raw is not None:
            arr = np.frombuffer(raw, dtype=dt.newbyteorder("<")).astype(dt)
        elif self.data_type == 1:
            arr = np.asarray(floats, dtype=dt)
        elif self.data_type == 11:
            arr = np.asarray(doubles, dtype=dt)
        elif self.data_type == 7:
            arr = np.asarray(int64s, dtype=dt)
        elif self.data_type in (12, 13):
            arr = np.asarray(uint64s, dtype=np.uint64).astype(dt)
        elif self.data_type == 10:   # fp16 travels as bit patterns in int32_data
            arr = np.asarray(int32s, dtype=np.uint16).view(np.float16)
        else:
            arr = np.asarray(int32s, dtype=np.int64).astype(dt)
        if arr.size != int(np.prod(shape, dtype=np.int64)):
            raise ProtoError("tensor %r: %d values for shape %s" % (self.name, arr.size, shape))
        self.array = arr.reshape(shape)


class AttributeProto:
    def __init__(self, buf: bytes):
        self.name = ""
        self.type = 0
        f = i = s = t = None
        floats, ints, strings = [], [], []
        for num, wt, v in fields(buf):
            if num == 1:
                self.name = v.decode("utf-8")
            elif num == 2:
                f = struct.unpack("<f", v)[0]
            elif num == 3:
                i = _signed(v)
            elif num == 4:
                s = bytes(v)
            elif num == 5:
                t = TensorProto(v)
            elif num == 7:
                floats += _packed_fixed(wt, v, "f", 4)
            elif num == 8:
                ints += _packed_varints(wt, v)
            elif num == 9:
                strings.append(bytes(v))
            elif num == 20:
                self.type = v
            elif num in (6, 10, 11):
                raise ProtoError("attribute %r holds a graph or tensor list, which is not supported" % self.name)
        # AttributeProto.AttributeType: FLOAT 1, INT 2, STRING 3, TENSOR 4, FLOATS 6, INTS 7, STRINGS 8
        kind = self.type
        if kind == 0:   # old exporters leave the type out
            kind = 1 if f is not None else 2 if i is not None else 3 if s is not None else 4 if t is not None else \
                6 if floats else 7 if ints else 8 if strings else 0
        self.value = {1: f if f is not None else 0.0, 2: i if i is not None else 0,
                      3: (s or b"").decode("utf-8"), 4: None if t is None else t.array, 6: floats, 7: ints,
                      8: [x.decode("utf-8") for x in strings]}.get(kind)
        if kind not in (1, 2, 3, 4, 6, 7, 8):
            raise ProtoError("attribute %r has unsupported type %d" % (self.name, kind))


class NodeProto:
    def __init__(self, buf: bytes):
        self.input: List[str] = []
        self.output: List[str] = []
        self.name = ""
        self.op_type = ""
        self.domain = ""
        self.attribute: List[AttributeProto] = []
        for num, wt, v in fields(buf):
            if num == 1:
                self.input.append(v.decode("utf-8"))
            elif num == 2:
                self.output.append(v.decode("utf-8"))
            elif num == 3:
                self.name = v.decode("utf-8")
            elif num == 4:
                self.op_type = v.decode("utf-8")
            elif num == 5:
                self.attribute.append(AttributeProto(v))
            elif num == 7:
                self.domain = v.decode("utf-8")


class ValueInfoProto:
    """name, elem_type (TensorProto.DataType, 0 if absent) and shape (None if absent; symbolic dims as str)."""
    def __init__(self, buf: bytes):
        self.name = ""
        self.elem_type = 0
        self.shape: Optional[List] = None
        for num, wt, v in fields(buf):
            if num == 1:
                self.name = v.decode("utf-8")
            elif num == 2:
                for n2, _, v2 in fields(v):          # TypeProto
                    if n2 != 1:
                        continue
                    for n3, _, v3 in fields(v2):     # TypeProto.Tensor
                        if n3 == 1:
                            self.elem_type = v3
                        elif n3 == 2:
                            self.shape = []
                            for n4, _, v4 in fields(v3):   # TensorShapeProto.dim
                                if n4 != 1:
                                    continue
                                dim: Any = None
                                for n5, _, v5 in fields(v4):
                                    if n5 == 1:
                                        dim = _signed(v5)
                                    elif n5 == 2:
                                        dim = v5.decode("utf-8")
                                self.shape.append(dim)


class GraphProto:
    def __init__(self, buf: bytes):
        self.name = ""
        self.node: List[NodeProto] = []
        self.initializer: List[TensorProto] = []
        self.input: List[ValueInfoProto] = []
        self.output: List[ValueInfoProto] = []
        self.value_info: List[ValueInfoProto] = []
        for num, wt, v in fields(buf):
            if num == 1:
                self.node.append(NodeProto(v))
            elif num == 2:
                self.name = v.decode("utf-8")
            elif num == 5:
                self.initializer.append(TensorProto(v))
            elif num == 11:
                self.input.append(ValueInfoProto(v))
            elif num == 12:
                self.output.append(ValueInfoProto(v))
            elif num == 13:
                self.value_info.append(ValueInfoProto(v))


class ModelProto:
    def __init__(self, buf: bytes):
        self.ir_version = 0
        self.producer_name = ""
        self.opset_import: Dict[str, int] = {}
        self.graph: Optional[GraphProto] = None
        for num, wt, v in fields(buf):
            if num == 1:
                self.ir_version = v
            elif num == 2:
                self.producer_name = v.decode("utf-8")
            elif num == 7:
                self.graph = GraphProto(v)
            elif num == 8:
                domain, version = "", 0
                for n2, _, v2 in fields(v):
                    if n2 == 1:
                        domain = v2.decode("utf-8")
                    elif n2 == 2:
                        version = v2
                self.opset_import[domain] = version
        if self.graph is None:
            raise ProtoError("not an ONNX model: no graph")


def load_model(source) -> ModelProto:
    """``source``: bytes, a path, or a file object."""
    if isinstance(source, (bytes, bytearray, memoryview)):
        data = bytes(source)
    elif hasattr(source, "read"):
        data = source.read()
    else:
        with open(source, "rb") as f:
            data = f.read()
    return ModelProto(data)
