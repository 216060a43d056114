"""ONNX Q/DQ -> operator graph, without the `onnx` package.

Mirrors the reference's importer (src/aie4ml/frontends/onnx/importer.py:31-130): the same 14 operators, the
same handler registry (`@onnx_handler(*op_types)` -> `fn(ctx, node, node_name, directives)`,
frontends/onnx/registry.py:12-34), the same lowering of QuantizeLinear / DequantizeLinear pairs to per-tensor
power-of-two QuantIntents (frontends/onnx/quantize.py), the same node kinds, roles and metadata, and the same
error messages. Differences: the file is decoded by onnx_proto (no protobuf dependency), static shapes come
from the small inference table below instead of onnx.shape_inference, and the result is a GPUModel.
"""

from __future__ import annotations

from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np

from ..aie_types import FloatFormat, FloatIntent, QuantIntent, RoundingMode, SaturationMode, is_float_intent
from ..ir import BackendContext, LogicalIR, OpNode, TensorVar, set_input_roles
from . import onnx_proto as op

OnnxHandler = Callable[['OnnxImportContext', op.Node, str, dict], None]
ONNX_HANDLERS: Dict[str, OnnxHandler] = {}


def onnx_handler(*op_types: str) -> Callable[[OnnxHandler], OnnxHandler]:
    """Register `fn` as the handler for one or more ONNX op types."""

    def register(fn: OnnxHandler) -> OnnxHandler:
        for t in op_types:
            if t in ONNX_HANDLERS:
                raise ValueError(f'duplicate ONNX handler for {t!r}: {ONNX_HANDLERS[t]} vs {fn}')
            ONNX_HANDLERS[t] = fn
        return fn

    return register


def dispatch(ctx: 'OnnxImportContext', node: op.Node, node_name: str, directives: dict) -> None:
    handler = ONNX_HANDLERS.get(node.op_type)
    if handler is None:
        raise ValueError(f'{node_name}: unsupported ONNX op {node.op_type}.')
    handler(ctx, node, node_name, directives)


# ---- helpers (frontends/onnx/utils.py) ------------------------------------------------------------------

def node_name_of(node: op.Node, index: int) -> str:
    name = (node.name or '').strip()
    return name if name else f'{node.op_type}_{index}'


def normalize_directives(name: str, raw: Any) -> Dict[str, Any]:
    """Keeps the directives that mean something on the GPU; the AIE placement / tiling / routing ones are
    accepted and dropped."""
    if raw is None:
        return {}
    if not isinstance(raw, dict):
        raise TypeError(f'{name}: layer directives must be a dict.')
    out: Dict[str, Any] = {}
    if 'approximation' in raw:
        out['approximation'] = str(raw['approximation'])
    if 'hccs' in raw:
        if not isinstance(raw['hccs'], dict):
            raise TypeError(f'{name}: hccs override must be a dict.')
        out['hccs'] = dict(raw['hccs'])
    if 'shift_per_channel' in raw:
        out['shift_per_channel'] = [int(s) for s in raw['shift_per_channel']]
    known = {'approximation', 'hccs', 'shift_per_channel', 'placement', 'microtiling', 'parallelism', 'io_route', 'layout'}
    unknown = sorted(set(raw) - known)
    if unknown:
        raise ValueError(f'{name}: unknown layer directives {unknown}.')
    return out


def scalar_tensor(initializers: Dict[str, np.ndarray], name: str, node_name: str) -> np.ndarray:
    if name not in initializers:
        raise ValueError(f'{node_name}: quantization parameter {name} must be an initializer.')
    arr = np.asarray(initializers[name])
    if arr.size != 1:
        raise ValueError(f'{node_name}: per-axis quantization is not supported for {name}.')
    return arr.reshape(())


def intent_from_qparams(initializers, scale_name: str, zero_name: str, qdtype, node_name: str) -> QuantIntent:
    """utils.py:187-217: symmetric (zero point 0), power-of-two scale, round-to-nearest-even, saturate."""
    scale = float(scalar_tensor(initializers, scale_name, node_name))
    zero = scalar_tensor(initializers, zero_name, node_name)
    if int(zero) != 0:
        raise ValueError(f'{node_name}: zero_point must be 0 for symmetric quantization.')
    dtype = np.dtype(qdtype)
    if not np.issubdtype(dtype, np.integer):
        raise ValueError(f'{node_name}: only integer quantization is supported; got {dtype}.')
    if scale <= 0.0:
        raise ValueError(f'{node_name}: quantization scale must be positive.')
    log2_scale = np.log2(scale)
    rounded = round(float(log2_scale))
    if not np.isclose(log2_scale, rounded, atol=1e-7):
        raise ValueError(f'{node_name}: scale {scale} is not a power of two.')
    return QuantIntent(width=int(dtype.itemsize * 8), frac=int(-rounded), signed=bool(np.issubdtype(dtype, np.signedinteger)),
                       rounding=RoundingMode.RND_CONV, saturation=SaturationMode.SAT)


def dequantize_data(data: np.ndarray, initializers, scale_name: str, zero_name: str, node_name: str) -> np.ndarray:
    scale = float(scalar_tensor(initializers, scale_name, node_name))
    zero = int(scalar_tensor(initializers, zero_name, node_name))
    return (np.asarray(data, dtype=np.float64) - float(zero)) * scale


def normalize_axis(axis: int, rank: int, node_name: str, op_type: str) -> int:
    normalized = axis + rank if axis < 0 else axis
    if not 0 <= normalized < rank:
        raise ValueError(f'{node_name}: {op_type} axis {axis} is out of range for rank {rank}.')
    return normalized


# ---- static shapes (replaces onnx.shape_inference for the supported operators) ----------------------------------

def _broadcast(a: Sequence[int], b: Sequence[int], what: str) -> Tuple[int, ...]:
    try:
        return tuple(int(x) for x in np.broadcast_shapes(tuple(a), tuple(b)))
    except ValueError as exc:
        raise ValueError(f'{what}: shapes {tuple(a)} and {tuple(b)} do not broadcast.') from exc


def build_shape_table(model: op.Model, initializers: Dict[str, np.ndarray], input_shapes: Dict[str, Tuple[int, ...]]):
    """Every tensor's static shape, keyed by ONNX value name (frontends/onnx/shapes.py:32-51)."""
    shape_of: Dict[str, Tuple[int, ...]] = {n: tuple(int(x) for x in np.asarray(a).shape) for n, a in initializers.items()}
    shape_of.update(input_shapes)
    for index, node in enumerate(model.graph.nodes):
        name = node_name_of(node, index)
        ins = [shape_of.get(i) for i in node.inputs]
        t = node.op_type
        if t not in ONNX_HANDLERS:
            continue  # dispatch reports it with the node's name
        if any(s is None for s, i in zip(ins, node.inputs) if i):
            continue  # an input without a shape: the handler's output_shape() raises
        if t in ('QuantizeLinear', 'DequantizeLinear', 'Relu', 'Softmax', 'LayerNormalization'):
            outs = [ins[0]]
        elif t in ('Add', 'Mul', 'Div'):
            outs = [_broadcast(ins[0], ins[1], name)]
        elif t == 'MatMul':
            a, b = ins
            if len(a) < 1 or len(b) < 1:
                raise ValueError(f'{name}: MatMul operands must have rank >= 1.')
            a2 = (1,) + tuple(a) if len(a) == 1 else tuple(a)
            b2 = tuple(b) + (1,) if len(b) == 1 else tuple(b)
            if a2[-1] != b2[-2]:
                raise ValueError(f'{name}: MatMul inner dimensions differ: {tuple(a)} x {tuple(b)}.')
            out = _broadcast(a2[:-2], b2[:-2], name) + (a2[-2], b2[-1])
            if len(b) == 1:
                out = out[:-1]
            if len(a) == 1:
                out = out[:-2] + out[-1:] if len(b) > 1 else out[:-1]
            outs = [out]
        elif t == 'Gemm':
            a, b = ins[0], ins[1]
            if len(a) != 2 or len(b) != 2:
                raise ValueError(f'{name}: Gemm operands must be rank-2.')
            m = a[1] if int(node.attrs.get('transA', 0)) else a[0]
            n = b[0] if int(node.attrs.get('transB', 0)) else b[1]
            outs = [(m, n)]
        elif t == 'Transpose':
            perm = node.attrs.get('perm') or list(reversed(range(len(ins[0]))))
            if sorted(int(p) for p in perm) != list(range(len(ins[0]))):
                raise ValueError(f'{name}: invalid permutation {list(perm)} for rank {len(ins[0])}.')
            outs = [tuple(ins[0][int(p)] for p in perm)]
        elif t == 'Concat':
            axis = normalize_axis(int(node.attrs.get('axis', -1)), len(ins[0]), name, 'Concat')
            outs = [tuple(sum(s[axis] for s in ins) if d == axis else ins[0][d] for d in range(len(ins[0])))]
        elif t == 'Split':
            src = ins[0]
            axis = normalize_axis(int(node.attrs.get('axis', 0)), len(src), name, 'Split')
            if len(node.inputs) == 2 and node.inputs[1] in initializers:
                sizes = [int(x) for x in np.asarray(initializers[node.inputs[1]]).reshape(-1)]
            elif node.attrs.get('split'):
                sizes = [int(x) for x in node.attrs['split']]
            else:
                sizes = [src[axis] // max(len(node.outputs), 1)] * len(node.outputs)
            outs = [tuple(sz if d == axis else src[d] for d in range(len(src))) for sz in sizes]
        elif t == 'Slice':
            src = list(ins[0])
            consts = [np.asarray(initializers[i]).reshape(-1) if i in initializers else None for i in node.inputs[1:]]
            if len(consts) >= 2 and consts[0] is not None and consts[1] is not None and consts[0].size == 1:
                axes = consts[2] if len(consts) >= 3 and consts[2] is not None else np.arange(1)
                axis = normalize_axis(int(axes[0]), len(src), name, 'Slice')
                start = max(0, min(src[axis], int(consts[0][0])))
                end = max(start, min(src[axis], int(consts[1][0])))
                src[axis] = end - start
            outs = [tuple(src)]
        else:  # pragma: no cover - every registered op is listed above
            continue
        for out_name, shape in zip(node.outputs, outs):
            if out_name:
                shape_of[out_name] = tuple(int(x) for x in shape)
    for vi in list(model.graph.value_info) + list(model.graph.outputs):  # declared shapes must agree
        if vi.shape is not None and all(d is not None for d in vi.shape) and vi.name in shape_of \
                and tuple(vi.shape) != shape_of[vi.name]:
            raise ValueError(f'{vi.name}: declared shape {tuple(vi.shape)} differs from the inferred {shape_of[vi.name]}.')
    return shape_of


# ---- import state (frontends/onnx/context.py) -----------------------------------------------------------------

# ONNX elem_type of a bare (not Q/DQ wrapped) graph input -> intent (frontends/onnx/context.py:18-24)
_FLOAT_INPUT_INTENT = {
    op.FLOAT: FloatIntent(width=32, format=FloatFormat.FP32),
    op.BFLOAT16: FloatIntent(width=16, format=FloatFormat.BF16),
    op.FLOAT8E4M3FN: FloatIntent(width=8, format=FloatFormat.FP8_E4M3),
}


class OnnxImportContext:
    """Mutable state threaded through the handler dispatch."""

    def __init__(self, backend: BackendContext, *, initializers, input_shapes, input_dtypes, shape_of, layer_directives):
        self.backend = backend
        self.graph: LogicalIR = backend.ir.logical
        self.device = backend.device
        self.initializers: Dict[str, np.ndarray] = initializers
        self.input_shapes: Dict[str, Tuple[int, ...]] = input_shapes
        self.input_dtypes: Dict[str, int] = input_dtypes
        self.shape_of: Dict[str, Tuple[int, ...]] = shape_of
        self.layer_directives: Dict[str, Any] = layer_directives
        self.used_directives: set = set()
        self.value_tensors: Dict[str, TensorVar] = {}   # ONNX value name -> lowered tensor
        self.q_aliases: Dict[str, Tuple[str, Any, QuantIntent, Tuple[int, ...]]] = {}  # Quantize output awaiting its Dequantize
        self.precision_mirrors: List[Tuple[str, str]] = []
        self.narrow_float_initializers: Dict[str, FloatFormat] = {}  # initializers the file stores as BFLOAT16 / FLOAT8E4M3FN

    def mirror_precision(self, target: str, source: str) -> None:
        self.precision_mirrors.append((target, source))

    def take_directives(self, node_name: str) -> Dict[str, Any]:
        directives = normalize_directives(node_name, self.layer_directives.get(node_name))
        if node_name in self.layer_directives:
            self.used_directives.add(node_name)
        return directives

    def output_shape(self, name: str, node_name: str) -> Tuple[int, ...]:
        if name not in self.shape_of:
            raise ValueError(f'{node_name}: shape inference produced no shape for {name!r}.')
        return tuple(int(x) for x in self.shape_of[name])

    def graph_input_tensor(self, name: str, shape: Sequence[int], intent: QuantIntent) -> TensorVar:
        tensor = self.graph.tensors.get(name)
        if tensor is None:
            tensor = TensorVar(name=name, shape=tuple(int(x) for x in shape), precision=intent)
            self.graph.add_tensor(tensor)
        elif tensor.precision is None:
            tensor.precision = intent
        elif tensor.precision != intent:
            raise ValueError(f'{name}: conflicting quantization intent for graph input.')
        return tensor

    def param_tensor(self, name: str, data: np.ndarray, intent: Optional[QuantIntent]) -> TensorVar:
        tensor = self.graph.tensors.get(name)
        arr = np.asarray(data, dtype=np.float64)
        if tensor is None:
            tensor = TensorVar(name=name, shape=tuple(int(x) for x in arr.shape), precision=intent, data=arr)
            self.graph.add_tensor(tensor)
            return tensor
        if tensor.data is None:
            raise ValueError(f'{name}: expected parameter tensor.')
        if tensor.precision != intent:
            raise ValueError(f'{name}: conflicting quantization intent for parameter tensor.')
        return tensor

    def source_for(self, name: str, node_name: str) -> TensorVar:
        """An activation tensor; never a constant."""
        if name in self.value_tensors:
            return self.value_tensors[name]
        if name in self.input_shapes:
            # a bare float graph input belongs to the float compute path (frontends/onnx/context.py:18-24, 131-143)
            intent = _FLOAT_INPUT_INTENT.get(self.input_dtypes.get(name))
            if intent is None:
                raise ValueError(f'{node_name}: graph input "{name}" has unsupported ONNX elem_type '
                                 f'{self.input_dtypes.get(name)}. Use QDQ wrapping for integer inputs.')
            tensor = self.graph_input_tensor(name, self.input_shapes[name], intent)
            self.bind(name, tensor)
            return tensor
        raise ValueError(f'{node_name}: unsupported input {name}. Expected a dequantized activation tensor.')

    def parameter_source_for(self, name: str, node_name: str) -> TensorVar:
        """A constant tensor: the result of a DequantizeLinear, or a float initializer."""
        if name in self.value_tensors:
            tensor = self.value_tensors[name]
            if not tensor.is_parameter:
                raise ValueError(f'{node_name}: parameter input {name} must be constant.')
            return tensor
        if name in self.initializers:
            data = np.asarray(self.initializers[name])
            if data.dtype not in (np.dtype(np.float32), np.dtype(np.float64)):
                raise ValueError(f'{node_name}: direct initializer inputs must be float32, or quantized via DequantizeLinear; '
                                 f'got {data.dtype}.')
            # a float constant: LayerNormalization scale / bias (the operator quantises those itself, whatever the
            # intent says) or a parameter of the float compute path (intent_from_initializer, utils.py:229-241)
            fmt = self.narrow_float_initializers.get(name, FloatFormat.FP32)
            width = {FloatFormat.BF16: 16, FloatFormat.FP8_E4M3: 8}.get(fmt, 32)
            return self.param_tensor(name, data, FloatIntent(width=width, format=fmt))
        raise ValueError(f'{node_name}: parameter input {name} must be a constant initializer.')

    def any_source_for(self, name: str, node_name: str) -> TensorVar:
        if name in self.value_tensors:
            return self.value_tensors[name]
        if name in self.initializers:
            return self.parameter_source_for(name, node_name)
        return self.source_for(name, node_name)

    def bind(self, name: str, tensor: TensorVar) -> None:
        self.value_tensors[name] = tensor

    def emit(self, op_type: str, node_name: str, *, inputs: Sequence[TensorVar],
             outputs: Sequence[Tuple[str, Sequence[int], Optional[Any]]], metadata: Dict[str, Any], directives: Dict[str, Any],
             roles: Optional[Sequence[str]] = None) -> OpNode:
        """Create a semantic OpNode, wire it, and register its outputs."""
        node = OpNode(name=f'{node_name}_aie', op_type=op_type, dialect=getattr(self.device, 'dialect', 'CDNA'))
        node.metadata.update(metadata)
        if roles is not None:
            node.metadata['input_roles'] = list(roles)
        node.directives.update(directives)
        for src in inputs:
            src.consumers.append(node)
        node.inputs.extend(inputs)
        for out_name, out_shape, out_precision in outputs:
            t = TensorVar(name=out_name, shape=tuple(int(x) for x in out_shape), precision=out_precision, producer=node)
            self.graph.add_tensor(t)
            node.outputs.append(t)
            self.value_tensors[out_name] = t
        self.graph.add_node(node)
        return node


# ---- QuantizeLinear / DequantizeLinear (frontends/onnx/quantize.py) ---------------------------------------------------

def _pin_if_unset(tensor, intent: QuantIntent, *, force_signed: bool) -> None:
    """Pin an un-quantized activation to a downstream Quantize's intent."""
    if tensor is None or tensor.is_parameter or tensor.precision is not None:
        return
    tensor.precision = QuantIntent(width=int(intent.width), frac=int(intent.frac), signed=True, rounding=intent.rounding,
                                   saturation=intent.saturation) if force_signed else intent


@onnx_handler('QuantizeLinear')
def _quantize_linear(ctx: OnnxImportContext, node: op.Node, node_name: str, _directives: dict) -> None:
    if len(node.inputs) != 3:
        raise ValueError(f'{node_name}: QuantizeLinear must have exactly 3 inputs.')
    src_name, scale_name, zero_name = node.inputs
    if zero_name not in ctx.initializers:
        raise ValueError(f'{node_name}: zero_point must be a constant initializer.')
    intent = intent_from_qparams(ctx.initializers, scale_name, zero_name, ctx.initializers[zero_name].dtype, node_name)
    out_name = node.outputs[0]
    if src_name in ctx.value_tensors:
        tensor = ctx.value_tensors[src_name]
        producer = tensor.producer
        relu = producer is not None and producer.op_type == 'activation' and producer.metadata.get('activation') == 'relu'
        if tensor.precision is None:
            if relu:
                _pin_if_unset(producer.inputs[0], intent, force_signed=True)
            elif producer is not None and producer.op_type == 'scale':
                _pin_if_unset(producer.inputs[0], intent, force_signed=False)
            elif producer is not None and producer.op_type == 'add':
                for inp in producer.inputs:  # a dense accumulator feeding a bias add carries the add's requant precision
                    _pin_if_unset(inp, intent, force_signed=False)
            tensor.precision = intent
        elif tensor.precision != intent:
            if not relu:
                raise ValueError(f'{node_name}: QuantizeLinear intent does not match source tensor precision.')
            _pin_if_unset(producer.inputs[0], intent, force_signed=True)
            tensor.precision = intent
        ctx.q_aliases[out_name] = ('tensor', tensor, intent, tuple(int(x) for x in tensor.shape))
    elif src_name in ctx.input_shapes:
        ctx.q_aliases[out_name] = ('input', src_name, intent, ctx.input_shapes[src_name])
    elif src_name in ctx.initializers:
        ctx.q_aliases[out_name] = ('initializer', src_name, intent, tuple(int(x) for x in ctx.initializers[src_name].shape))
    else:
        raise ValueError(f'{node_name}: QuantizeLinear input {src_name} is unsupported.')


_ONNX_INT_ELEM_TYPE_TO_NP = {op.UINT8: np.uint8, op.INT8: np.int8, op.UINT16: np.uint16, op.INT16: np.int16,
                             op.INT32: np.int32, op.INT64: np.int64}


@onnx_handler('DequantizeLinear')
def _dequantize_linear(ctx: OnnxImportContext, node: op.Node, node_name: str, _directives: dict) -> None:
    if len(node.inputs) != 3:
        raise ValueError(f'{node_name}: DequantizeLinear must have exactly 3 inputs.')
    src_name, scale_name, zero_name = node.inputs
    out_name = node.outputs[0]
    if zero_name not in ctx.initializers:
        raise ValueError(f'{node_name}: zero_point must be a constant initializer.')
    if src_name in ctx.q_aliases:
        kind, ref, q_intent, src_shape = ctx.q_aliases[src_name]
        intent = intent_from_qparams(ctx.initializers, scale_name, zero_name, ctx.initializers[zero_name].dtype, node_name)
        if intent != q_intent:
            raise ValueError(f'{node_name}: QuantizeLinear/DequantizeLinear parameters do not match.')
        if kind == 'tensor':
            tensor = ref
        elif kind == 'input':
            tensor = ctx.graph_input_tensor(ref, src_shape, intent)
        else:
            tensor = ctx.param_tensor(ref, dequantize_data(ctx.initializers[ref], ctx.initializers, scale_name, zero_name,
                                                           node_name), intent)
        ctx.bind(out_name, tensor)
    elif src_name in ctx.initializers:
        intent = intent_from_qparams(ctx.initializers, scale_name, zero_name, ctx.initializers[src_name].dtype, node_name)
        ctx.bind(out_name, ctx.param_tensor(src_name, dequantize_data(ctx.initializers[src_name], ctx.initializers, scale_name,
                                                                      zero_name, node_name), intent))
    elif src_name in ctx.input_shapes:
        raw = _ONNX_INT_ELEM_TYPE_TO_NP.get(ctx.input_dtypes[src_name])
        if raw is None:
            raise ValueError(f'{node_name}: direct DequantizeLinear on graph input requires integer input type.')
        intent = intent_from_qparams(ctx.initializers, scale_name, zero_name, raw, node_name)
        ctx.bind(out_name, ctx.graph_input_tensor(src_name, ctx.input_shapes[src_name], intent))
    else:
        raise ValueError(f'{node_name}: DequantizeLinear input {src_name} is unsupported.')


# ---- MatMul / Gemm (handlers/matmul.py) -------------------------------------------------------------------------------

def _mm_meta(layer_class: str, source_class: str, n_in: int, n_out: int, node_name: str) -> dict:
    return {'n_in': n_in, 'n_out': n_out, 'use_bias': False, 'layer_class': layer_class, 'source_class': source_class,
            'source_layer': node_name}


@onnx_handler('MatMul', 'Gemm')
def _matmul_gemm(ctx: OnnxImportContext, node: op.Node, node_name: str, directives: dict) -> None:
    kind = node.op_type
    if kind == 'MatMul':
        if len(node.inputs) != 2:
            raise ValueError(f'{node_name}: MatMul must have exactly 2 inputs.')
        lhs_name, rhs_name = node.inputs
        bias_name, trans_b = None, False
        rhs_const = rhs_name in ctx.initializers or (rhs_name in ctx.value_tensors and ctx.value_tensors[rhs_name].is_parameter)
    else:
        if len(node.inputs) not in (2, 3):
            raise ValueError(f'{node_name}: Gemm must have 2 or 3 inputs.')
        if float(node.attrs.get('alpha', 1.0)) != 1.0:
            raise ValueError(f'{node_name}: Gemm alpha must be 1.')
        if float(node.attrs.get('beta', 1.0)) != 1.0:
            raise ValueError(f'{node_name}: Gemm beta must be 1.')
        if int(node.attrs.get('transA', 0)) != 0:
            raise ValueError(f'{node_name}: Gemm transA is not supported.')
        lhs_name, rhs_name = node.inputs[:2]
        bias_name = node.inputs[2] if len(node.inputs) == 3 and node.inputs[2] else None
        trans_b = int(node.attrs.get('transB', 0)) == 1
        rhs_const = True
    lhs = ctx.source_for(lhs_name, node_name)
    if lhs.is_parameter:
        raise ValueError(f'{node_name}: activation input cannot be constant.')
    out_name = node.outputs[0]
    out_shape = ctx.output_shape(out_name, node_name)
    out_precision = lhs.precision if is_float_intent(lhs.precision) else None  # handlers/matmul.py:51

    if not rhs_const:
        rhs = ctx.source_for(rhs_name, node_name)
        rs = ctx.output_shape(rhs_name, node_name)
        n_in, n_out = int(rs[0] if len(rs) == 1 else rs[-2]), int(1 if len(rs) == 1 else rs[-1])
        ctx.emit('matmul', node_name, inputs=[lhs, rhs], outputs=[(out_name, out_shape, out_precision)], roles=['lhs', 'rhs'],
                 metadata=_mm_meta('MatMul', 'MatMul', n_in, n_out, node_name), directives=directives)
        return

    rhs = ctx.parameter_source_for(rhs_name, node_name)
    data = np.asarray(rhs.data, dtype=np.float64)
    if trans_b:
        data = np.transpose(data)
    if data.ndim != 2:
        if kind == 'Gemm':
            raise ValueError(f'{node_name}: ONNX Gemm weight matrix must be rank-2.')
        n_in, n_out = int(data.shape[0] if data.ndim == 1 else data.shape[-2]), int(1 if data.ndim == 1 else data.shape[-1])
        ctx.emit('matmul', node_name, inputs=[lhs, ctx.param_tensor(f'{node_name}_rhs', data, rhs.precision)],
                 outputs=[(out_name, out_shape, out_precision)], roles=['lhs', 'rhs'],
                 metadata=_mm_meta('MatMul', 'MatMul', n_in, n_out, node_name), directives=directives)
        return
    n_in, n_out = int(data.shape[0]), int(data.shape[1])
    weight = ctx.param_tensor(f'{node_name}_weight', data, rhs.precision)
    if bias_name is None:
        ctx.emit('dense', node_name, inputs=[lhs, weight], outputs=[(out_name, out_shape, out_precision)], roles=['lhs', 'rhs'],
                 metadata=_mm_meta('Dense', kind, n_in, n_out, node_name), directives=directives)
        return
    # Gemm with bias: dense -> add(bias); the bias-folding pass re-fuses the add into the dense
    prebias = f'{node_name}_prebias'
    ctx.mirror_precision(prebias, out_name)
    ctx.emit('dense', node_name, inputs=[lhs, weight], outputs=[(prebias, out_shape, out_precision)], roles=['lhs', 'rhs'],
             metadata=_mm_meta('Dense', kind, n_in, n_out, node_name), directives=directives)
    bias = ctx.parameter_source_for(bias_name, node_name)
    bias_data = np.asarray(bias.data, dtype=np.float64).reshape(-1)
    if int(bias_data.size) != n_out:
        raise ValueError(f'{node_name}: Gemm bias must contain exactly {n_out} elements.')
    ctx.emit('add', f'{node_name}_bias', inputs=[ctx.value_tensors[prebias], ctx.param_tensor(f'{node_name}_bias', bias_data,
                                                                                             bias.precision)],
             outputs=[(out_name, out_shape, out_precision)], roles=['lhs', 'rhs'],
             metadata={'layer_class': 'Add', 'source_class': 'Gemm', 'source_layer': node_name}, directives={})


# ---- elementwise, activation, normalisation (handlers/elementwise.py, activation.py, norm.py) -------------------------

@onnx_handler('Mul', 'Div')
def _mul_div(ctx: OnnxImportContext, node: op.Node, node_name: str, directives: dict) -> None:
    kind = node.op_type
    if len(node.inputs) != 2:
        raise ValueError(f'{node_name}: {kind} must have exactly 2 inputs.')
    if kind == 'Mul':
        consts = [n for n in node.inputs if n in ctx.initializers]
        if len(consts) != 1:
            raise NotImplementedError(f'{node_name}: Mul currently requires exactly one constant input.')
        const_name = consts[0]
        src_name = node.inputs[1] if node.inputs[0] == const_name else node.inputs[0]
        scale = float(np.asarray(ctx.initializers[const_name]).reshape(-1)[0])
    else:
        src_name, const_name = node.inputs
        if const_name not in ctx.initializers:
            raise NotImplementedError(f'{node_name}: Div currently requires a constant divisor.')
        divisor = float(np.asarray(ctx.initializers[const_name]).reshape(-1)[0])
        if divisor == 0.0:
            raise ValueError(f'{node_name}: Div constant divisor must be nonzero.')
        scale = 1.0 / divisor
    if np.asarray(ctx.initializers[const_name]).size != 1:
        raise NotImplementedError(f'{node_name}: {kind} currently requires a scalar constant.')
    src = ctx.source_for(src_name, node_name)
    out_name = node.outputs[0]
    ctx.emit('scale', node_name, inputs=[src], outputs=[(out_name, ctx.output_shape(out_name, node_name), src.precision)],
             roles=['lhs'], metadata={'scale': scale, 'layer_class': kind, 'source_class': kind, 'source_layer': node_name},
             directives=directives)


@onnx_handler('Add')
def _add(ctx: OnnxImportContext, node: op.Node, node_name: str, directives: dict) -> None:
    if len(node.inputs) != 2:
        raise ValueError(f'{node_name}: Add must have exactly 2 inputs.')
    lhs_name, rhs_name = node.inputs
    lhs, rhs = ctx.any_source_for(lhs_name, node_name), ctx.any_source_for(rhs_name, node_name)
    out_name = node.outputs[0]
    # a constant addend is a bias candidate; two activations must be exact-shape (the add kernel does not broadcast)
    if lhs.is_parameter == rhs.is_parameter:
        ls, rs = ctx.output_shape(lhs_name, node_name), ctx.output_shape(rhs_name, node_name)
        if ls != rs:
            raise ValueError(f'{node_name}: generic Add only supports exact-shape elementwise inputs; got {ls} and {rs}.')
    out_precision = lhs.precision if is_float_intent(lhs.precision) else None  # handlers/elementwise.py:61
    ctx.emit('add', node_name, inputs=[lhs, rhs], outputs=[(out_name, ctx.output_shape(out_name, node_name), out_precision)],
             roles=['lhs', 'rhs'], metadata={'layer_class': 'Add', 'source_class': 'Add', 'source_layer': node_name},
             directives=directives)


@onnx_handler('Relu')
def _relu(ctx: OnnxImportContext, node: op.Node, node_name: str, directives: dict) -> None:
    if len(node.inputs) != 1:
        raise ValueError(f'{node_name}: Relu must have exactly 1 input.')
    src = ctx.source_for(node.inputs[0], node_name)
    out_name = node.outputs[0]
    ctx.emit('activation', node_name, inputs=[src], outputs=[(out_name, ctx.output_shape(out_name, node_name), src.precision)],
             roles=['lhs'], metadata={'activation': 'relu', 'layer_class': 'Activation', 'source_layer': node_name},
             directives=directives)


@onnx_handler('LayerNormalization')
def _layer_norm(ctx: OnnxImportContext, node: op.Node, node_name: str, directives: dict) -> None:
    if len(node.inputs) not in (2, 3):
        raise ValueError(f'{node_name}: LayerNormalization must have 2 or 3 inputs.')
    x_name, scale_name = node.inputs[0], node.inputs[1]
    bias_name = node.inputs[2] if len(node.inputs) == 3 and node.inputs[2] else None
    x_shape = ctx.output_shape(x_name, node_name)
    axis = normalize_axis(int(node.attrs.get('axis', -1)), len(x_shape), node_name, 'LayerNormalization')
    x = ctx.source_for(x_name, node_name)
    gamma = ctx.parameter_source_for(scale_name, node_name)
    if bias_name is not None:
        beta = ctx.parameter_source_for(bias_name, node_name)
    else:
        beta = ctx.param_tensor(f'{node_name}_beta_zero', np.zeros(tuple(x_shape[axis:]), dtype=np.float64), gamma.precision)
    ctx.emit('layer_norm', node_name, inputs=[x, gamma, beta],
             outputs=[(node.outputs[0], ctx.output_shape(node.outputs[0], node_name), None)], roles=['lhs', 'gamma', 'beta'],
             metadata={'layer_class': 'LayerNormalization', 'source_class': 'LayerNormalization', 'source_layer': node_name,
                       'epsilon': float(node.attrs.get('epsilon', 1e-5)), 'axis': axis}, directives=directives)


@onnx_handler('Softmax')
def _softmax(ctx: OnnxImportContext, node: op.Node, node_name: str, directives: dict) -> None:
    if len(node.inputs) != 1:
        raise ValueError(f'{node_name}: Softmax must have exactly 1 input.')
    src = ctx.source_for(node.inputs[0], node_name)
    in_shape = ctx.output_shape(node.inputs[0], node_name)
    axis = normalize_axis(int(node.attrs.get('axis', -1)), len(in_shape), node_name, 'Softmax')
    out_name = node.outputs[0]
    ctx.emit('softmax', node_name, inputs=[src], outputs=[(out_name, ctx.output_shape(out_name, node_name), None)],
             roles=['lhs'], metadata={'axis': axis, 'layer_class': 'Softmax', 'source_class': 'Softmax', 'source_layer': node_name},
             directives=directives)


# ---- shape / view operators (handlers/tensor.py) ---------------------------------------------------------------------

@onnx_handler('Transpose')
def _transpose(ctx: OnnxImportContext, node: op.Node, node_name: str, directives: dict) -> None:
    if len(node.inputs) != 1:
        raise ValueError(f'{node_name}: Transpose must have exactly 1 input.')
    src = ctx.any_source_for(node.inputs[0], node_name)
    in_shape = ctx.output_shape(node.inputs[0], node_name)
    perm = [int(x) for x in (node.attrs.get('perm') or reversed(range(len(in_shape))))]
    if sorted(perm) != list(range(len(in_shape))):
        raise ValueError(f'{node_name}: invalid permutation {perm} for rank {len(in_shape)}.')
    out_name = node.outputs[0]
    if src.is_parameter:
        ctx.bind(out_name, ctx.param_tensor(out_name, np.transpose(np.asarray(src.data, dtype=np.float64), axes=perm), src.precision))
        return
    ctx.emit('transpose', node_name, inputs=[src], outputs=[(out_name, ctx.output_shape(out_name, node_name), src.precision)],
             roles=['lhs'], metadata={'perm': perm, 'data_format': 'channels_last', 'layer_class': 'Transpose',
                                      'source_layer': node_name}, directives=directives)


@onnx_handler('Slice', 'Split')
def _slice_split(ctx: OnnxImportContext, node: op.Node, node_name: str, directives: dict) -> None:
    kind = node.op_type
    src_name = node.inputs[0]
    src_shape = ctx.output_shape(src_name, node_name)
    if kind == 'Slice':
        if len(node.inputs) not in (3, 4, 5):
            raise ValueError(f'{node_name}: Slice must have 3 to 5 inputs.')
        for n in node.inputs[1:]:
            if n and n not in ctx.initializers:
                raise NotImplementedError(f'{node_name}: Slice parameters must be constant initializers.')
        arr = lambda i: np.asarray(ctx.initializers[node.inputs[i]], dtype=np.int64).reshape(-1)  # noqa: E731
        starts, ends = arr(1), arr(2)
        axes = arr(3) if len(node.inputs) >= 4 and node.inputs[3] else np.arange(starts.size, dtype=np.int64)
        steps = arr(4) if len(node.inputs) >= 5 and node.inputs[4] else np.ones(starts.size, dtype=np.int64)
        if starts.size != 1 or ends.size != 1 or axes.size != 1 or steps.size != 1:
            raise NotImplementedError(f'{node_name}: Slice currently supports exactly one sliced axis.')
        if int(steps[0]) != 1:
            raise NotImplementedError(f'{node_name}: Slice currently supports only unit steps.')
        axis = normalize_axis(int(axes[0]), len(src_shape), node_name, 'Slice')
        start = max(0, min(int(src_shape[axis]), int(starts[0])))
        end = max(start, min(int(src_shape[axis]), int(ends[0])))
        ranges = [(start, end - start)]
    else:
        if len(node.inputs) not in (1, 2):
            raise ValueError(f'{node_name}: Split must have 1 or 2 inputs.')
        axis = normalize_axis(int(node.attrs.get('axis', 0)), len(src_shape), node_name, 'Split')
        if len(node.inputs) == 2 and node.inputs[1]:
            if node.inputs[1] not in ctx.initializers:
                raise NotImplementedError(f'{node_name}: Split sizes must be a constant initializer.')
            sizes = [int(x) for x in np.asarray(ctx.initializers[node.inputs[1]], dtype=np.int64).reshape(-1)]
        else:
            sizes = [int(x) for x in list(node.attrs.get('split') or [])]
            if not sizes:
                if int(src_shape[axis]) % len(node.outputs) != 0:
                    raise ValueError(f'{node_name}: equal Split does not divide axis {axis} exactly.')
                sizes = [int(src_shape[axis]) // len(node.outputs)] * len(node.outputs)
        if len(sizes) != len(node.outputs) or any(s <= 0 for s in sizes):
            raise ValueError(f'{node_name}: Split sizes must be positive and match output count.')
        if sum(sizes) != int(src_shape[axis]):
            raise ValueError(f'{node_name}: Split sizes must cover axis {axis} exactly.')
        ranges, offset = [], 0
        for s in sizes:
            ranges.append((offset, s))
            offset += s
    src = ctx.source_for(src_name, node_name)
    ctx.emit(kind.lower(), node_name, inputs=[src],
             outputs=[(o, ctx.output_shape(o, node_name), src.precision) for o in node.outputs], roles=['lhs'],
             metadata={'axis': axis, 'slices': [{'start': s, 'extent': e} for s, e in ranges], 'layer_class': kind,
                       'source_class': kind, 'source_layer': node_name}, directives=directives)


@onnx_handler('Concat')
def _concat(ctx: OnnxImportContext, node: op.Node, node_name: str, directives: dict) -> None:
    if len(node.inputs) < 1:
        raise ValueError(f'{node_name}: Concat must have at least one input.')
    sources = [ctx.source_for(n, node_name) for n in node.inputs]
    if any(s.is_parameter for s in sources):
        raise ValueError(f'{node_name}: Concat currently supports activation tensors only.')
    shapes = [ctx.output_shape(n, node_name) for n in node.inputs]
    rank = len(shapes[0])
    if rank < 1:
        raise ValueError(f'{node_name}: Concat does not accept scalar inputs.')
    if any(len(s) != rank for s in shapes):
        raise ValueError(f'{node_name}: Concat inputs must have the same rank.')
    axis = normalize_axis(int(node.attrs.get('axis', -1)), rank, node_name, 'Concat')
    for s in shapes[1:]:
        if tuple(s[:axis]) != tuple(shapes[0][:axis]) or tuple(s[axis + 1:]) != tuple(shapes[0][axis + 1:]):
            raise ValueError(f'{node_name}: Concat input shapes disagree outside axis {axis}: {shapes}.')
    for s in sources[1:]:
        if s.precision != sources[0].precision:
            raise ValueError(f'{node_name}: Concat inputs must use identical precision contracts.')
    ctx.emit('concat', node_name, inputs=sources,
             outputs=[(node.outputs[0], ctx.output_shape(node.outputs[0], node_name), sources[0].precision)],
             metadata={'axis': axis, 'layer_class': 'Concat', 'source_class': 'Concat', 'source_layer': node_name},
             directives=directives)


# ---- driver (frontends/onnx/importer.py) ------------------------------------------------------------------------------

def lower_onnx_model(model_or_path, config: Optional[Dict[str, Any]] = None) -> BackendContext:
    model = op.load_model(model_or_path)
    config = dict(config or {})
    backend = BackendContext(config=config)
    graph = backend.ir.logical
    initializers = {t.name: np.asarray(t.array) for t in model.graph.initializers}
    narrow = {t.name: (FloatFormat.BF16 if t.bfloat16 else FloatFormat.FP8_E4M3) for t in model.graph.initializers
              if t.bfloat16 or t.float8}
    input_shapes: Dict[str, Tuple[int, ...]] = {}
    input_dtypes: Dict[str, int] = {}
    for vi in model.graph.inputs:
        if vi.name in initializers:
            continue
        if vi.shape is None:
            raise ValueError(f'{vi.name}: tensor shape is missing.')
        if any(d is None for d in vi.shape):
            raise ValueError(f'{vi.name}: dynamic shapes are not supported.')
        if not vi.shape:
            raise ValueError(f'{vi.name}: scalar inputs are not supported.')
        input_shapes[vi.name] = tuple(int(d) for d in vi.shape)
        input_dtypes[vi.name] = int(vi.elem_type)
    for name, shape in input_shapes.items():
        graph.add_tensor(TensorVar(name=name, shape=shape, precision=None))
        graph.mark_graph_input(name)

    ctx = OnnxImportContext(backend, initializers=initializers, input_shapes=input_shapes, input_dtypes=input_dtypes,
                            shape_of=build_shape_table(model, initializers, input_shapes),
                            layer_directives=dict(config.get('LayerDirectives', {}) or {}))
    ctx.narrow_float_initializers = narrow
    for index, node in enumerate(model.graph.nodes):
        name = node_name_of(node, index)
        dispatch(ctx, node, name, ctx.take_directives(name))
    _finalize(ctx, model.graph)
    return backend


def _finalize(ctx: OnnxImportContext, graph_proto: op.Graph) -> None:
    graph = ctx.graph
    unused = sorted(set(ctx.layer_directives) - ctx.used_directives)
    if unused:
        raise ValueError('Unused LayerDirectives entries: ' + ', '.join(unused))
    for output in graph_proto.outputs:
        if output.name not in ctx.value_tensors:
            raise ValueError(f'Graph output {output.name}: expected a lowered semantic tensor.')
        tensor = ctx.value_tensors[output.name]
        if output.name not in graph.tensors:  # the output is the Dequantize alias of a tensor known by another name
            graph.tensors.pop(tensor.name, None)
            tensor.name = output.name
            graph.tensors[output.name] = tensor
        graph.mark_graph_output(output.name)
    for node in graph.nodes:
        roles = list(node.metadata.get('input_roles') or [])
        if roles:
            set_input_roles(node, node.inputs, roles)
    for target, source in ctx.precision_mirrors:
        t, o = graph.tensors.get(target), graph.tensors.get(source)
        if t is not None and t.precision is None and o is not None:
            t.precision = o.precision
    for t in graph.tensors.values():
        if not t.is_parameter and t.precision is None:
            raise ValueError(f'{t.name}: missing quantization intent after ONNX QDQ lowering.')


def from_onnx(model_or_path, config: Optional[Dict[str, Any]] = None):
    """ONNX Q/DQ model (path, bytes or onnx_proto.Model) -> GPUModel (frontends/onnx/importer.py:113-130)."""
    from ..model import GPUModel

    return GPUModel.from_context(lower_onnx_model(model_or_path, config), source_model=model_or_path)
