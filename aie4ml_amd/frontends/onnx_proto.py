"""A self-contained reader and writer for the part of the ONNX file format the importer needs.

The reference loads models with the `onnx` package (src/aie4ml/frontends/onnx/utils.py:17-23,
importer.py:40-46); that package is not a dependency here. An .onnx file is a protobuf-encoded ModelProto;
this module decodes the wire format directly (varints, length-delimited fields, packed and unpacked repeated
scalars) into small dataclasses, and encodes them back, for the messages and fields of onnx.proto that a
Q/DQ graph of the 14 supported operators uses. Unknown fields are skipped on read.
"""

from __future__ import annotations

import struct
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Dict, List, Optional, Tuple, Union

import numpy as np

# TensorProto.DataType
FLOAT, UINT8, INT8, UINT16, INT16, INT32, INT64, BOOL, FLOAT16, DOUBLE = 1, 2, 3, 4, 5, 6, 7, 9, 10, 11
BFLOAT16, FLOAT8E4M3FN = 16, 17  # no numpy dtype: held as float32 arrays and flagged (Tensor.bfloat16 / .float8)
NP_OF = {FLOAT: np.float32, UINT8: np.uint8, INT8: np.int8, UINT16: np.uint16, INT16: np.int16, INT32: np.int32,
         INT64: np.int64, BOOL: np.bool_, FLOAT16: np.float16, DOUBLE: np.float64}
ONNX_OF = {np.dtype(v): k for k, v in NP_OF.items()}


@dataclass
class Tensor:
    name: str
    array: np.ndarray
    bfloat16: bool = False  # the file stores (or shall store) the values as ONNX BFLOAT16
    float8: bool = False    # ... as ONNX FLOAT8E4M3FN


@dataclass
class ValueInfo:
    name: str
    elem_type: int = 0
    shape: Optional[Tuple[Optional[int], ...]] = None  # None entries: symbolic dimensions


@dataclass
class Node:
    op_type: str
    inputs: List[str] = field(default_factory=list)
    outputs: List[str] = field(default_factory=list)
    name: str = ''
    attrs: Dict[str, Any] = field(default_factory=dict)
    domain: str = ''


@dataclass
class Graph:
    name: str = ''
    nodes: List[Node] = field(default_factory=list)
    initializers: List[Tensor] = field(default_factory=list)
    inputs: List[ValueInfo] = field(default_factory=list)
    outputs: List[ValueInfo] = field(default_factory=list)
    value_info: List[ValueInfo] = field(default_factory=list)


@dataclass
class Model:
    graph: Graph = field(default_factory=Graph)
    ir_version: int = 8
    opset: Dict[str, int] = field(default_factory=lambda: {'': 17})
    producer_name: str = ''


# ---- wire format: decode ------------------------------------------------------------------------------

def _varint(buf: bytes, pos: int) -> Tuple[int, int]:
    result = shift = 0
    while True:
        if pos >= len(buf):
            raise ValueError('truncated varint')
        b = buf[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7
        if shift > 70:
            raise ValueError('varint too long')


def _signed64(v: int) -> int:
    v &= (1 << 64) - 1
    return v - (1 << 64) if v >> 63 else v


def _fields(buf: bytes):
    """Yields (field number, wire type, value); value is an int (varint / fixed) or a bytes slice."""
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
            n, pos = _varint(buf, pos)
            val = buf[pos:pos + n]
            if len(val) != n:
                raise ValueError('truncated length-delimited field')
            pos += n
        elif wt == 5:
            val = buf[pos:pos + 4]
            pos += 4
        else:
            raise ValueError(f'unsupported protobuf wire type {wt}')
        yield num, wt, val


def _ints(wt: int, val, out: List[int]) -> None:
    """A repeated int64 field arrives one varint at a time or packed into one length-delimited blob."""
    if wt == 0:
        out.append(_signed64(val))
    else:
        pos = 0
        while pos < len(val):
            v, pos = _varint(val, pos)
            out.append(_signed64(v))


def _floats(wt: int, val, out: List[float], fmt: str = '<f') -> None:
    size = struct.calcsize(fmt)
    for off in range(0, len(val), size):
        out.append(struct.unpack_from(fmt, val, off)[0])


def _parse_tensor(buf: bytes) -> Tensor:
    dims: List[int] = []
    dtype, name, raw = 0, '', None
    f32: List[float] = []
    f64: List[float] = []
    i32: List[int] = []
    i64: List[int] = []
    u64: List[int] = []
    for num, wt, val in _fields(buf):
        if num == 1:
            _ints(wt, val, dims)
        elif num == 2:
            dtype = val
        elif num == 4:
            _floats(wt, val, f32)
        elif num == 5:
            _ints(wt, val, i32)
        elif num == 7:
            _ints(wt, val, i64)
        elif num == 8:
            name = val.decode()
        elif num == 9:
            raw = bytes(val)
        elif num == 10:
            _floats(wt, val, f64, '<d')
        elif num == 11:
            _ints(wt, val, u64)
        elif num == 13 and len(val):
            raise NotImplementedError(f'tensor {name!r}: external data is not supported')
    if dtype == BFLOAT16:  # 16-bit patterns in raw_data or int32_data; widened to float32 (exact)
        bits = np.frombuffer(raw, dtype='<u2') if raw is not None else np.array(i32, dtype=np.int64)
        arr = (bits.astype(np.uint32) << 16).view(np.float32)
        count = int(np.prod(dims)) if dims else 1
        if arr.size != count:
            raise ValueError(f'tensor {name!r}: {arr.size} values for shape {tuple(dims)}')
        return Tensor(name, arr.reshape(tuple(dims)), bfloat16=True)
    if dtype == FLOAT8E4M3FN:  # codes in raw_data or int32_data; decoded to float32 (exact)
        codes = np.frombuffer(raw, dtype=np.uint8) if raw is not None else np.array(i32, dtype=np.int64).astype(np.uint8)
        arr = _fp8_decode(codes)
        count = int(np.prod(dims)) if dims else 1
        if arr.size != count:
            raise ValueError(f'tensor {name!r}: {arr.size} values for shape {tuple(dims)}')
        return Tensor(name, arr.reshape(tuple(dims)), float8=True)
    if dtype not in NP_OF:
        raise NotImplementedError(f'tensor {name!r}: ONNX data type {dtype} is not supported')
    npdt = np.dtype(NP_OF[dtype])
    if raw is not None:
        arr = np.frombuffer(raw, dtype=npdt.newbyteorder('<')).astype(npdt)
    elif dtype == FLOAT:
        arr = np.array(f32, dtype=npdt)
    elif dtype == DOUBLE:
        arr = np.array(f64, dtype=npdt)
    elif dtype == INT64:
        arr = np.array(i64, dtype=npdt)
    elif dtype == FLOAT16:
        arr = np.array(i32, dtype=np.uint16).view(np.float16)
    else:  # the narrow integer types and bool travel in int32_data
        arr = np.array(i32, dtype=np.int64).astype(npdt)
    count = int(np.prod(dims)) if dims else 1
    if arr.size != count:
        raise ValueError(f'tensor {name!r}: {arr.size} values for shape {tuple(dims)}')
    return Tensor(name, arr.reshape(tuple(dims)))


def _parse_value_info(buf: bytes) -> ValueInfo:
    vi = ValueInfo('')
    for num, _wt, val in _fields(buf):
        if num == 1:
            vi.name = val.decode()
        elif num == 2:  # TypeProto
            for n2, _w2, v2 in _fields(val):
                if n2 != 1:  # tensor_type
                    continue
                for n3, _w3, v3 in _fields(v2):
                    if n3 == 1:
                        vi.elem_type = v3
                    elif n3 == 2:  # TensorShapeProto
                        dims: List[Optional[int]] = []
                        for n4, _w4, v4 in _fields(v3):
                            if n4 != 1:
                                continue
                            d: Optional[int] = None
                            for n5, _w5, v5 in _fields(v4):
                                if n5 == 1:
                                    d = _signed64(v5)
                            dims.append(d)
                        vi.shape = tuple(dims)
    return vi


def _parse_attribute(buf: bytes) -> Tuple[str, Any]:
    name, atype = '', 0
    f = i = s = t = None
    fl: List[float] = []
    il: List[int] = []
    sl: List[bytes] = []
    for num, wt, val in _fields(buf):
        if num == 1:
            name = val.decode()
        elif num == 2:
            f = struct.unpack('<f', val)[0]
        elif num == 3:
            i = _signed64(val)
        elif num == 4:
            s = bytes(val)
        elif num == 5:
            t = _parse_tensor(val)
        elif num == 7:
            _floats(wt, val, fl)
        elif num == 8:
            _ints(wt, val, il)
        elif num == 9:
            sl.append(bytes(val))
        elif num == 20:
            atype = val
    if atype == 0:  # writers before IR version 3 left the type out: infer it from what is present
        atype = 1 if f is not None else 2 if i is not None else 3 if s is not None else 4 if t is not None else \
            6 if fl else 7 if il else 8 if sl else 0
    value = {1: f, 2: i, 3: s.decode() if s is not None else None, 4: t, 6: fl, 7: il,
             8: [x.decode() for x in sl]}.get(atype)
    if atype not in (1, 2, 3, 4, 6, 7, 8):
        raise NotImplementedError(f'attribute {name!r}: type {atype} is not supported')
    return name, value


def _parse_node(buf: bytes) -> Node:
    node = Node('')
    for num, _wt, val in _fields(buf):
        if num == 1:
            node.inputs.append(val.decode())
        elif num == 2:
            node.outputs.append(val.decode())
        elif num == 3:
            node.name = val.decode()
        elif num == 4:
            node.op_type = val.decode()
        elif num == 5:
            k, v = _parse_attribute(val)
            node.attrs[k] = v
        elif num == 7:
            node.domain = val.decode()
    return node


def _parse_graph(buf: bytes) -> Graph:
    g = Graph()
    for num, _wt, val in _fields(buf):
        if num == 1:
            g.nodes.append(_parse_node(val))
        elif num == 2:
            g.name = val.decode()
        elif num == 5:
            g.initializers.append(_parse_tensor(val))
        elif num == 11:
            g.inputs.append(_parse_value_info(val))
        elif num == 12:
            g.outputs.append(_parse_value_info(val))
        elif num == 13:
            g.value_info.append(_parse_value_info(val))
        elif num == 15 and len(val):
            raise NotImplementedError('sparse initializers are not supported')
    return g


def parse_model(data: bytes) -> Model:
    m = Model(opset={})
    seen_graph = False
    for num, _wt, val in _fields(data):
        if num == 1:
            m.ir_version = val
        elif num == 2:
            m.producer_name = val.decode()
        elif num == 7:
            m.graph = _parse_graph(val)
            seen_graph = True
        elif num == 8:
            domain, version = '', 0
            for n2, _w2, v2 in _fields(val):
                if n2 == 1:
                    domain = v2.decode()
                elif n2 == 2:
                    version = v2
            m.opset[domain] = version
    if not seen_graph:
        raise ValueError('not an ONNX model: no graph field')
    return m


def load_model(source: Union[str, Path, bytes, Model]) -> Model:
    if isinstance(source, Model):
        return source
    if isinstance(source, (bytes, bytearray, memoryview)):
        return parse_model(bytes(source))
    return parse_model(Path(source).read_bytes())


# ---- wire format: encode ------------------------------------------------------------------------------

def _enc_varint(v: int) -> bytes:
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


def _key(num: int, wt: int) -> bytes:
    return _enc_varint((num << 3) | wt)


def _ld(num: int, payload: bytes) -> bytes:
    return _key(num, 2) + _enc_varint(len(payload)) + payload


def _vi(num: int, v: int) -> bytes:
    return _key(num, 0) + _enc_varint(v)


def _packed_ints(num: int, values) -> bytes:
    return _ld(num, b''.join(_enc_varint(int(v)) for v in values)) if len(values) else b''


def _fp8_decode(codes: np.ndarray) -> np.ndarray:
    """FLOAT8E4M3FN codes -> float32: bias 7, subnormals m * 2^-9, no infinities, S.1111.111 is NaN."""
    c = codes.astype(np.int64)
    e, m = (c >> 3) & 0xF, c & 7
    mag = np.where(e == 0, m * 2.0 ** -9, (1.0 + m / 8.0) * np.exp2(e - 7.0))
    mag = np.where((e == 15) & (m == 7), np.nan, mag)
    return np.where(c & 0x80, -mag, mag).astype(np.float32)


_FP8_VALUES = None


def _fp8_encode_exact(values: np.ndarray, name: str) -> np.ndarray:
    """Values that are exact in FLOAT8E4M3FN -> their codes (table lookup; anything else is an error)."""
    global _FP8_VALUES
    if _FP8_VALUES is None:
        table = _fp8_decode(np.arange(256, dtype=np.uint8))
        _FP8_VALUES = {float(v): c for c, v in enumerate(table.tolist()) if v == v and not (c == 0x80)}
    flat = values.reshape(-1).tolist()
    try:
        return np.array([_FP8_VALUES[float(v) + 0.0] for v in flat], dtype=np.uint8)
    except KeyError as exc:
        raise ValueError(f'tensor {name!r}: value {exc.args[0]} is not exact in float8 e4m3') from None


def _ser_tensor(t: Tensor) -> bytes:
    arr = np.ascontiguousarray(t.array)
    if t.bfloat16:
        bits = np.ascontiguousarray(arr, dtype=np.float32).view(np.uint32)
        if np.any(bits & 0xFFFF):
            raise ValueError(f'tensor {t.name!r}: values are not exact in bfloat16')
        out = _packed_ints(1, arr.shape) + _vi(2, BFLOAT16) + _ld(8, t.name.encode())
        return out + _ld(9, (bits >> 16).astype('<u2').tobytes())
    if t.float8:
        codes = _fp8_encode_exact(np.ascontiguousarray(arr, dtype=np.float32), t.name)
        return _packed_ints(1, arr.shape) + _vi(2, FLOAT8E4M3FN) + _ld(8, t.name.encode()) + _ld(9, codes.tobytes())
    if arr.dtype not in ONNX_OF:
        raise NotImplementedError(f'tensor {t.name!r}: dtype {arr.dtype} has no ONNX type here')
    out = _packed_ints(1, arr.shape) + _vi(2, ONNX_OF[arr.dtype]) + _ld(8, t.name.encode())
    return out + _ld(9, arr.astype(arr.dtype.newbyteorder('<')).tobytes())


def _ser_value_info(v: ValueInfo) -> bytes:
    tensor_type = _vi(1, v.elem_type)
    if v.shape is not None:
        dims = b''.join(_ld(1, _vi(1, d) if d is not None else _ld(2, b'?')) for d in v.shape)
        tensor_type += _ld(2, dims)
    return _ld(1, v.name.encode()) + _ld(2, _ld(1, tensor_type))


def _ser_attribute(name: str, value: Any) -> bytes:
    out = _ld(1, name.encode())
    if isinstance(value, bool) or isinstance(value, (int, np.integer)):
        return out + _vi(3, int(value)) + _vi(20, 2)
    if isinstance(value, (float, np.floating)):
        return out + _key(2, 5) + struct.pack('<f', float(value)) + _vi(20, 1)
    if isinstance(value, str):
        return out + _ld(4, value.encode()) + _vi(20, 3)
    if isinstance(value, Tensor):
        return out + _ld(5, _ser_tensor(value)) + _vi(20, 4)
    seq = list(value)
    if seq and all(isinstance(x, (float, np.floating)) for x in seq):
        return out + _ld(7, b''.join(struct.pack('<f', float(x)) for x in seq)) + _vi(20, 6)
    if all(isinstance(x, (int, np.integer)) for x in seq):
        return out + _packed_ints(8, seq) + _vi(20, 7)
    raise NotImplementedError(f'attribute {name!r}: unsupported value {value!r}')


def _ser_node(n: Node) -> bytes:
    out = b''.join(_ld(1, s.encode()) for s in n.inputs) + b''.join(_ld(2, s.encode()) for s in n.outputs)
    out += _ld(3, n.name.encode()) + _ld(4, n.op_type.encode())
    out += b''.join(_ld(5, _ser_attribute(k, v)) for k, v in n.attrs.items())
    if n.domain:
        out += _ld(7, n.domain.encode())
    return out


def serialize_model(m: Model) -> bytes:
    g = m.graph
    graph = b''.join(_ld(1, _ser_node(n)) for n in g.nodes) + _ld(2, g.name.encode())
    graph += b''.join(_ld(5, _ser_tensor(t)) for t in g.initializers)
    graph += b''.join(_ld(11, _ser_value_info(v)) for v in g.inputs)
    graph += b''.join(_ld(12, _ser_value_info(v)) for v in g.outputs)
    graph += b''.join(_ld(13, _ser_value_info(v)) for v in g.value_info)
    out = _vi(1, m.ir_version)
    if m.producer_name:
        out += _ld(2, m.producer_name.encode())
    out += _ld(7, graph)
    for domain, version in m.opset.items():
        out += _ld(8, _ld(1, domain.encode()) + _vi(2, version))
    return out


def save_model(m: Model, path: Union[str, Path]) -> None:
    Path(path).write_bytes(serialize_model(m))
