"""A float64 evaluator of ONNX models, written from the ONNX operator definitions and the protobuf wire format only.

It is the independent side of the float-simulation check (the semantics of the reference's
scripts/check_onnx_bit_exact.py:128-136, where onnxruntime plays this part): it reads the same .onnx bytes as
`aie4ml_amd.from_onnx`, but shares no code with the importer, the passes, the operator resolution or the protobuf
reader of the package. Nothing here knows about shifts, accumulators or integer kernels: QuantizeLinear divides by the
scale, rounds half to even and saturates; everything else is plain float64 numpy.

Operators: QuantizeLinear, DequantizeLinear, MatMul, Gemm, Add, Mul, Div, Relu, Transpose, Split, Slice, Concat,
Softmax, LayerNormalization.
"""

from __future__ import annotations

import struct

import numpy as np

# ---- protobuf wire format ----------------------------------------------------------------------------------------


def _varint(buf, pos):
    out, shift = 0, 0
    while True:
        b = buf[pos]
        pos += 1
        out |= (b & 0x7F) << shift
        if b < 0x80:
            return out, pos
        shift += 7


def _walk(buf):
    """Yields (field number, wire type, value) for one message: ints for varint / fixed, bytes for length-delimited."""
    pos, n = 0, len(buf)
    while pos < n:
        key, pos = _varint(buf, pos)
        num, wt = key >> 3, key & 7
        if wt == 0:
            val, pos = _varint(buf, pos)
        elif wt == 1:
            val, pos = buf[pos:pos + 8], pos + 8
        elif wt == 2:
            ln, pos = _varint(buf, pos)
            val, pos = buf[pos:pos + ln], pos + ln
        elif wt == 5:
            val, pos = buf[pos:pos + 4], pos + 4
        else:
            raise ValueError(f'wire type {wt}')
        yield num, wt, val


def _s64(v):
    return v - (1 << 64) if v >= (1 << 63) else v


def _repeated_ints(wt, val):
    if wt == 0:
        return [_s64(val)]
    out, pos = [], 0
    while pos < len(val):
        v, pos = _varint(val, pos)
        out.append(_s64(v))
    return out


# TensorProto.DataType -> numpy
_DT = {1: np.float32, 2: np.uint8, 3: np.int8, 4: np.uint16, 5: np.int16, 6: np.int32, 7: np.int64, 11: np.float64,
       12: np.uint32, 13: np.uint64}


def _tensor(buf):
    dims, dtype, name, raw = [], None, '', None
    f32, i32, i64, f64 = [], [], [], []
    for num, wt, val in _walk(buf):
        if num == 1:
            dims += _repeated_ints(wt, val)
        elif num == 2:
            dtype = val
        elif num == 8:
            name = val.decode()
        elif num == 9:
            raw = bytes(val)
        elif num == 4:
            f32 += list(struct.unpack(f'<{len(val) // 4}f', val)) if wt == 2 else [struct.unpack('<f', val)[0]]
        elif num == 5:
            i32 += _repeated_ints(wt, val)
        elif num == 7:
            i64 += _repeated_ints(wt, val)
        elif num == 10:
            f64 += list(struct.unpack(f'<{len(val) // 8}d', val)) if wt == 2 else [struct.unpack('<d', val)[0]]
    np_dt = _DT[dtype]
    if raw is not None:
        arr = np.frombuffer(raw, dtype=np.dtype(np_dt).newbyteorder('<')).astype(np_dt)
    else:
        arr = np.array(f32 or i32 or i64 or f64, dtype=np_dt)
    return name, arr.reshape(dims)


def _attribute(buf):
    name, out = '', None
    ints, floats = [], []
    for num, wt, val in _walk(buf):
        if num == 1:
            name = val.decode()
        elif num == 2:
            out = struct.unpack('<f', val)[0]
        elif num == 3:
            out = _s64(val)
        elif num == 4:
            out = bytes(val)
        elif num == 5:
            out = _tensor(val)[1]
        elif num == 7:
            floats += list(struct.unpack(f'<{len(val) // 4}f', val)) if wt == 2 else [struct.unpack('<f', val)[0]]
        elif num == 8:
            ints += _repeated_ints(wt, val)
    if out is None:
        out = ints if ints else floats
    return name, out


def _node(buf):
    n = {'in': [], 'out': [], 'name': '', 'op': '', 'attr': {}}
    for num, _wt, val in _walk(buf):
        if num == 1:
            n['in'].append(val.decode())
        elif num == 2:
            n['out'].append(val.decode())
        elif num == 3:
            n['name'] = val.decode()
        elif num == 4:
            n['op'] = val.decode()
        elif num == 5:
            k, v = _attribute(val)
            n['attr'][k] = v
    return n


def _value_name(buf):
    for num, _wt, val in _walk(buf):
        if num == 1:
            return val.decode()
    return ''


def parse(data: bytes):
    """-> (nodes in file order, initializers, graph input names, graph output names)"""
    graph = None
    for num, _wt, val in _walk(data):
        if num == 7:
            graph = val
    nodes, inits, inputs, outputs = [], {}, [], []
    for num, _wt, val in _walk(graph):
        if num == 1:
            nodes.append(_node(val))
        elif num == 5:
            name, arr = _tensor(val)
            inits[name] = arr
        elif num == 11:
            inputs.append(_value_name(val))
        elif num == 12:
            outputs.append(_value_name(val))
    return nodes, inits, [i for i in inputs if i not in inits], outputs


# ---- operator definitions (ONNX operator set 17) --------------------------------------------------------------------


def _quantize_linear(x, scale, zp):
    info = np.iinfo(zp.dtype)
    q = np.rint(np.asarray(x, dtype=np.float64) / np.asarray(scale, np.float64)) + np.asarray(zp, np.float64)  # rint: half to even
    return np.clip(q, info.min, info.max).astype(zp.dtype)


def _dequantize_linear(x, scale, zp):
    return (np.asarray(x, dtype=np.float64) - np.asarray(zp, np.float64)) * np.asarray(scale, np.float64)


def _softmax(x, axis):
    e = np.exp(x - np.max(x, axis=axis, keepdims=True))
    return e / np.sum(e, axis=axis, keepdims=True)


def _layer_norm(x, scale, bias, axis, eps):
    axes = tuple(range(axis % x.ndim, x.ndim))
    mean = np.mean(x, axis=axes, keepdims=True)
    var = np.mean((x - mean) ** 2, axis=axes, keepdims=True)
    y = (x - mean) / np.sqrt(var + eps) * scale
    return y if bias is None else y + bias


def _split(x, sizes, axis, n_out):
    if sizes is None:
        sizes = [x.shape[axis] // n_out] * n_out
    edges = np.cumsum([0] + [int(s) for s in sizes])
    idx = [slice(None)] * x.ndim
    out = []
    for a, b in zip(edges[:-1], edges[1:]):
        idx[axis] = slice(int(a), int(b))
        out.append(x[tuple(idx)])
    return out


def _slice(x, starts, ends, axes, steps):
    axes = list(range(len(starts))) if axes is None else [int(a) for a in axes]
    steps = [1] * len(starts) if steps is None else [int(s) for s in steps]
    idx = [slice(None)] * x.ndim
    for s, e, a, st in zip(starts, ends, axes, steps):
        idx[a % x.ndim] = slice(int(s), int(e), st)  # Python slicing clamps out-of-range ends the way ONNX asks
    return x[tuple(idx)]


def run(data: bytes, feeds: dict) -> dict:
    """Evaluates the model in float64. `feeds`: graph input name -> array. Returns graph output name -> array."""
    nodes, inits, inputs, outputs = parse(data)
    env = dict(inits)
    for name in inputs:
        env[name] = np.asarray(feeds[name], dtype=np.float64)
    for n in nodes:
        a = n['attr']
        x = [env[i] if i else None for i in n['in']]
        op = n['op']
        if op == 'QuantizeLinear':
            y = [_quantize_linear(x[0], x[1], x[2])]
        elif op == 'DequantizeLinear':
            y = [_dequantize_linear(x[0], x[1], x[2] if len(x) > 2 else np.zeros((), x[0].dtype))]
        elif op == 'MatMul':
            y = [np.matmul(np.asarray(x[0], np.float64), np.asarray(x[1], np.float64))]
        elif op == 'Gemm':
            A = x[0].T if a.get('transA', 0) else x[0]
            B = x[1].T if a.get('transB', 0) else x[1]
            r = float(a.get('alpha', 1.0)) * (np.asarray(A, np.float64) @ np.asarray(B, np.float64))
            if len(x) > 2 and x[2] is not None:
                r = r + float(a.get('beta', 1.0)) * np.asarray(x[2], np.float64)
            y = [r]
        elif op == 'Add':
            y = [np.asarray(x[0], np.float64) + np.asarray(x[1], np.float64)]
        elif op == 'Mul':
            y = [np.asarray(x[0], np.float64) * np.asarray(x[1], np.float64)]
        elif op == 'Div':
            y = [np.asarray(x[0], np.float64) / np.asarray(x[1], np.float64)]
        elif op == 'Relu':
            y = [np.maximum(x[0], 0)]
        elif op == 'Transpose':
            y = [np.transpose(x[0], a.get('perm') or None)]
        elif op == 'Split':
            sizes = x[1] if len(x) > 1 and x[1] is not None else a.get('split')
            y = _split(x[0], sizes, int(a.get('axis', 0)) % x[0].ndim, len(n['out']))
        elif op == 'Slice':
            y = [_slice(x[0], x[1], x[2], x[3] if len(x) > 3 else None, x[4] if len(x) > 4 else None)]
        elif op == 'Concat':
            y = [np.concatenate(x, axis=int(a['axis']))]
        elif op == 'Softmax':
            y = [_softmax(np.asarray(x[0], np.float64), int(a.get('axis', -1)))]
        elif op == 'LayerNormalization':
            y = [_layer_norm(np.asarray(x[0], np.float64), np.asarray(x[1], np.float64),
                             None if len(x) < 3 or x[2] is None else np.asarray(x[2], np.float64),
                             int(a.get('axis', -1)), float(a.get('epsilon', 1e-5)))]
        else:
            raise NotImplementedError(f'{n["name"]}: ONNX operator {op}')
        for name, val in zip(n['out'], y):
            env[name] = val
    return {o: env[o] for o in outputs}


def requantize_output(values, width: int, signed: bool, frac: int):
    """Float graph output -> the integer grid of the executor's output tensor (round half to even, saturate): what the
    reference's checker does to onnxruntime's outputs before it compares (scripts/check_onnx_bit_exact.py:38-47)."""
    q = np.rint(np.asarray(values, dtype=np.float64) * float(1 << frac) if frac >= 0 else np.asarray(values, np.float64) / float(1 << -frac))
    lo, hi = (-(1 << (width - 1)), (1 << (width - 1)) - 1) if signed else (0, (1 << width) - 1)
    return np.clip(q, lo, hi).astype(np.int64)
