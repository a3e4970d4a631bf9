"""Dependency-free writer of ONNX model files.

The reference downloads its models and simplifies them with onnx/onnxsim at
build time (reference cmake/models.cmake:13-95); neither package nor any
network exists here, so graphs are produced by this module: a small protobuf
wire encoder for the messages FluidML's parser reads (ModelProto, GraphProto,
NodeProto, AttributeProto, TensorProto, ValueInfoProto; field numbers of
onnx/onnx.proto) and a `GraphBuilder` that records a static shape for every
value, because the reference takes intermediate shapes from graph.value_info
only (reference src/worker/parser.cpp:246-248) and infers none.
"""
from __future__ import annotations

import struct
from typing import Dict, Iterable, List, Optional, Sequence, Tuple, Union

import numpy as np

# TensorProto.DataType
FLOAT, INT32, INT64, BOOL = 1, 6, 7, 9
NP_TO_ONNX = {np.dtype(np.float32): FLOAT, np.dtype(np.int32): INT32, np.dtype(np.int64): INT64, np.dtype(np.bool_): BOOL}
ONNX_TO_NP = {v: k for k, v in NP_TO_ONNX.items()}

# AttributeProto.AttributeType
ATTR_FLOAT, ATTR_INT, ATTR_STRING, ATTR_TENSOR, ATTR_FLOATS, ATTR_INTS = 1, 2, 3, 4, 6, 7


# ---------------------------------------------------------------- wire encoding

def _varint(value: int) -> bytes:
    if value < 0:
        value += 1 << 64  # two's complement, 10 bytes
    out = bytearray()
    while True:
        byte = value & 0x7F
        value >>= 7
        if value:
            out.append(byte | 0x80)
        else:
            out.append(byte)
            return bytes(out)


def _key(field: int, wire: int) -> bytes:
    return _varint((field << 3) | wire)


def _f_varint(field: int, value: int) -> bytes:
    return _key(field, 0) + _varint(int(value))


def _f_bytes(field: int, payload: bytes) -> bytes:
    return _key(field, 2) + _varint(len(payload)) + payload


def _f_string(field: int, text: str) -> bytes:
    return _f_bytes(field, text.encode("utf-8"))


def _f_float(field: int, value: float) -> bytes:
    return _key(field, 5) + struct.pack("<f", float(value))


def _f_packed_varints(field: int, values: Iterable[int]) -> bytes:
    return _f_bytes(field, b"".join(_varint(int(v)) for v in values))


def encode_tensor(name: str, array: np.ndarray) -> bytes:
    """TensorProto with raw_data (dims=1, data_type=2, name=8, raw_data=9)."""
    array = np.asarray(array)
    dtype = NP_TO_ONNX[array.dtype]
    out = b""
    if array.ndim:
        out += _f_packed_varints(1, array.shape)
    out += _f_varint(2, dtype)
    out += _f_string(8, name)
    out += _f_bytes(9, np.ascontiguousarray(array).tobytes())
    return out


def encode_attribute(name: str, value) -> bytes:
    """AttributeProto (name=1, f=2, i=3, t=5, floats=7, ints=8, type=20)."""
    out = _f_string(1, name)
    if isinstance(value, bool):
        out += _f_varint(3, int(value)) + _f_varint(20, ATTR_INT)
    elif isinstance(value, (int, np.integer)):
        out += _f_varint(3, int(value)) + _f_varint(20, ATTR_INT)
    elif isinstance(value, (float, np.floating)):
        out += _f_float(2, float(value)) + _f_varint(20, ATTR_FLOAT)
    elif isinstance(value, np.ndarray):
        out += _f_bytes(5, encode_tensor("", value)) + _f_varint(20, ATTR_TENSOR)
    elif isinstance(value, (list, tuple)) and all(isinstance(v, (int, np.integer)) for v in value):
        out += _f_packed_varints(8, value) + _f_varint(20, ATTR_INTS)
    else:
        raise TypeError(f"attribute {name}: unsupported value {value!r}")
    return out


def encode_value_info(name: str, elem_type: int, shape: Sequence[int]) -> bytes:
    """ValueInfoProto{name=1, type=2{tensor_type=1{elem_type=1, shape=2{dim=1{dim_value=1}}}}}."""
    dims = b"".join(_f_bytes(1, _f_varint(1, d)) for d in shape)
    tensor_type = _f_varint(1, elem_type) + _f_bytes(2, dims)
    return _f_string(1, name) + _f_bytes(2, _f_bytes(1, tensor_type))


def encode_node(op_type: str, name: str, inputs: Sequence[str], outputs: Sequence[str], attrs: Dict[str, object]) -> bytes:
    """NodeProto (input=1, output=2, name=3, op_type=4, attribute=5)."""
    out = b"".join(_f_string(1, i) for i in inputs)
    out += b"".join(_f_string(2, o) for o in outputs)
    out += _f_string(3, name) + _f_string(4, op_type)
    out += b"".join(_f_bytes(5, encode_attribute(k, v)) for k, v in attrs.items())
    return out


# ---------------------------------------------------------------- graph builder

class Value:
    """A named tensor of the graph under construction."""

    def __init__(self, name: str, dtype, shape: Sequence[int], const: Optional[np.ndarray] = None):
        self.name = name
        self.dtype = np.dtype(dtype)
        self.shape = tuple(int(s) for s in shape)
        self.const = const

    def __repr__(self):
        return f"Value({self.name}, {self.dtype}, {self.shape})"


class NodeRecord:
    def __init__(self, op_type: str, name: str, inputs: List[Value], outputs: List[Value], attrs: Dict[str, object]):
        self.op_type, self.name, self.inputs, self.outputs, self.attrs = op_type, name, inputs, outputs, attrs


class GraphBuilder:
    """Collects inputs, initializers and nodes; every node output gets a static shape."""

    def __init__(self, name: str = "graph", opset: int = 17):
        self.name = name
        self.opset = opset
        self.inputs: List[Value] = []
        self.outputs: List[Value] = []
        self.initializers: List[Value] = []
        self.nodes: List[NodeRecord] = []
        self._counter = 0
        self._names = set()

    def _fresh(self, hint: str) -> str:
        while True:
            self._counter += 1
            name = f"{hint}_{self._counter}"
            if name not in self._names:
                self._names.add(name)
                return name

    def input(self, name: str, dtype, shape: Sequence[int]) -> Value:
        v = Value(name, dtype, shape)
        self._names.add(name)
        self.inputs.append(v)
        return v

    def const(self, array, name: Optional[str] = None) -> Value:
        """Initializer; a rank-0 array becomes what FluidML treats as a scalar operand."""
        array = np.asarray(array)
        name = name or self._fresh("const")
        self._names.add(name)
        v = Value(name, array.dtype, array.shape, const=array)
        self.initializers.append(v)
        return v

    def scalar(self, value, dtype=np.float32, name: Optional[str] = None) -> Value:
        return self.const(np.array(value, dtype=dtype), name)

    def node(self, op_type: str, inputs: Sequence[Value], out_shape: Sequence[int], out_dtype=None,
             name: Optional[str] = None, out_name: Optional[str] = None, **attrs) -> Value:
        name = name or self._fresh(op_type)
        self._names.add(name)
        out_dtype = np.dtype(out_dtype) if out_dtype is not None else inputs[0].dtype
        out = Value(out_name or self._fresh(op_type.lower() + "_out"), out_dtype, out_shape)
        self._names.add(out.name)
        self.nodes.append(NodeRecord(op_type, name, list(inputs), [out], dict(attrs)))
        return out

    def output(self, value: Value) -> Value:
        self.outputs.append(value)
        return value

    def serialize(self) -> bytes:
        out_names = {v.name for v in self.outputs}
        parts = [_f_bytes(1, encode_node(n.op_type, n.name, [i.name for i in n.inputs], [o.name for o in n.outputs],
                                         n.attrs)) for n in self.nodes]
        parts.append(_f_string(2, self.name))
        parts += [_f_bytes(5, encode_tensor(v.name, v.const)) for v in self.initializers]
        parts += [_f_bytes(11, encode_value_info(v.name, NP_TO_ONNX[v.dtype], v.shape)) for v in self.inputs]
        parts += [_f_bytes(12, encode_value_info(v.name, NP_TO_ONNX[v.dtype], v.shape)) for v in self.outputs]
        for n in self.nodes:
            for o in n.outputs:
                if o.name not in out_names:
                    parts.append(_f_bytes(13, encode_value_info(o.name, NP_TO_ONNX[o.dtype], o.shape)))
        graph_len = sum(len(p) for p in parts)
        opset = _f_string(1, "") + _f_varint(2, self.opset)
        head = _f_varint(1, 8) + _f_string(2, "fluidml_amd.onnx_writer")  # ir_version, producer_name
        return b"".join([head, _key(7, 2), _varint(graph_len)] + parts + [_f_bytes(8, opset)])

    def save(self, path: str) -> str:
        with open(path, "wb") as f:
            f.write(self.serialize())
        return path
