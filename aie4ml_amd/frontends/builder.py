"""Programmatic graph construction: emits the same node kinds, roles, metadata and traits the reference's
ONNX handlers emit (src/aie4ml/frontends/onnx/handlers/*.py), for use where no ONNX / hls4ml package is
available. Tensors are float-valued parameters plus QuantIntent precisions, exactly as after import; the
fold / fuse passes then run on the result unchanged.
"""

from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np

from ..aie_types import QuantIntent, RoundingMode, SaturationMode
from ..ir import BackendContext, OpNode, TensorVar, set_input_roles


def qint(width: int, frac: int, signed: bool = True, rounding: RoundingMode = RoundingMode.RND_CONV,
         saturation: SaturationMode = SaturationMode.SAT) -> QuantIntent:
    return QuantIntent(width=width, frac=frac, signed=signed, rounding=rounding, saturation=saturation)


class GraphBuilder:
    def __init__(self, config: Optional[Dict] = None):
        self.ctx = BackendContext(config=dict(config or {}))
        self.graph = self.ctx.ir.logical
        self._n = 0

    # ---- tensors
    def _uid(self, prefix: str) -> str:
        self._n += 1
        return f'{prefix}_{self._n}'

    def input(self, name: str, shape: Sequence[int], precision: QuantIntent) -> TensorVar:
        t = TensorVar(name=name, shape=tuple(int(s) for s in shape), precision=precision)
        self.graph.add_tensor(t)
        self.graph.mark_graph_input(name)
        return t

    def param(self, name: str, data, precision: Optional[QuantIntent]) -> TensorVar:
        arr = np.asarray(data, dtype=np.float64)
        t = TensorVar(name=name, shape=tuple(arr.shape), precision=precision, data=arr)
        self.graph.add_tensor(t)
        return t

    def output(self, tensor: TensorVar) -> TensorVar:
        self.graph.mark_graph_output(tensor.name)
        return tensor

    def _emit(self, op_type: str, name: str, inputs: List[TensorVar], outputs: List[Tuple[str, Tuple[int, ...], Optional[QuantIntent]]],
              roles: Iterable[str], metadata: Dict, directives: Optional[Dict] = None) -> List[TensorVar]:
        node = OpNode(name=f'{name}_aie', op_type=op_type, metadata=dict(metadata), directives=dict(directives or {}))
        node.inputs = list(inputs)
        for t in inputs:
            t.consumers.append(node)
        outs = []
        for oname, oshape, oprec in outputs:
            t = TensorVar(name=oname, shape=tuple(int(s) for s in oshape), precision=oprec, producer=node)
            self.graph.add_tensor(t)
            outs.append(t)
        node.outputs = outs
        set_input_roles(node, inputs, list(roles))
        self.graph.add_node(node)
        return outs

    # ---- operators (what the ONNX handlers emit before any folding)
    def dense(self, x: TensorVar, weight, w_precision: QuantIntent, out_precision: QuantIntent, bias=None,
              bias_precision: Optional[QuantIntent] = None, relu: bool = False, name: Optional[str] = None,
              directives: Optional[Dict] = None) -> TensorVar:
        """MatMul/Gemm with a constant rank-2 RHS: dense (+ add for the bias, + activation for ReLU)."""
        name = name or self._uid('dense')
        W = np.asarray(weight, dtype=np.float64)
        n_in, n_out = int(W.shape[0]), int(W.shape[1])
        wt = self.param(f'{name}_weight', W, w_precision)
        oshape = tuple(x.shape[:-1]) + (n_out,)
        meta = {'n_in': n_in, 'n_out': n_out, 'use_bias': False, 'layer_class': 'Dense', 'source_class': 'Gemm',
                'source_layer': name}
        first_out = f'{name}_prebias' if bias is not None else (f'{name}_prerelu' if relu else f'{name}_out')
        (y,) = self._emit('dense', name, [x, wt], [(first_out, oshape, out_precision)], ['lhs', 'rhs'], meta, directives)
        if bias is not None:
            bt = self.param(f'{name}_bias', np.asarray(bias, dtype=np.float64).reshape(-1), bias_precision)
            nxt = f'{name}_prerelu' if relu else f'{name}_out'
            (y,) = self._emit('add', f'{name}_bias', [y, bt], [(nxt, oshape, out_precision)], ['lhs', 'rhs'],
                              {'layer_class': 'Add', 'source_class': 'Gemm', 'source_layer': name})
        if relu:
            (y,) = self._emit('activation', f'{name}_relu', [y], [(f'{name}_out', oshape, out_precision)], ['lhs'],
                              {'activation': 'relu', 'layer_class': 'Activation', 'source_layer': name})
        return y

    def matmul(self, a: TensorVar, b: TensorVar, out_precision: QuantIntent, name: Optional[str] = None) -> TensorVar:
        name = name or self._uid('matmul')
        n_in, n_out = int(b.shape[-2]), int(b.shape[-1])
        oshape = tuple(a.shape[:-1]) + (n_out,)
        meta = {'n_in': n_in, 'n_out': n_out, 'use_bias': False, 'layer_class': 'MatMul', 'source_class': 'MatMul',
                'source_layer': name}
        (y,) = self._emit('matmul', name, [a, b], [(f'{name}_out', oshape, out_precision)], ['lhs', 'rhs'], meta)
        return y

    def transpose(self, x: TensorVar, perm: Sequence[int], name: Optional[str] = None) -> TensorVar:
        name = name or self._uid('transpose')
        oshape = tuple(x.shape[p] for p in perm)
        (y,) = self._emit('transpose', name, [x], [(f'{name}_out', oshape, x.precision)], ['lhs'],
                          {'perm': [int(p) for p in perm], 'data_format': 'channels_last', 'layer_class': 'Transpose'})
        return y

    def split(self, x: TensorVar, axis: int, sizes: Sequence[int], name: Optional[str] = None) -> List[TensorVar]:
        name = name or self._uid('split')
        ax = axis + len(x.shape) if axis < 0 else axis
        outs, slices, start = [], [], 0
        for i, sz in enumerate(sizes):
            shape = list(x.shape)
            shape[ax] = int(sz)
            outs.append((f'{name}_out{i}', tuple(shape), x.precision))
            slices.append({'start': start, 'extent': int(sz)})
            start += int(sz)
        return self._emit('split', name, [x], outs, ['lhs'], {'axis': ax, 'slices': slices, 'layer_class': 'Split'})

    def concat(self, xs: Sequence[TensorVar], axis: int, name: Optional[str] = None) -> TensorVar:
        name = name or self._uid('concat')
        ax = axis + len(xs[0].shape) if axis < 0 else axis
        shape = list(xs[0].shape)
        shape[ax] = sum(int(t.shape[ax]) for t in xs)
        (y,) = self._emit('concat', name, list(xs), [(f'{name}_out', tuple(shape), xs[0].precision)],
                          [f'in{i}' for i in range(len(xs))], {'axis': ax, 'layer_class': 'Concat'})
        return y

    def scale(self, x: TensorVar, scale: float, out_precision: Optional[QuantIntent] = None, name: Optional[str] = None) -> TensorVar:
        """Mul / Div by a positive constant (folded into a neighbour by FoldScale)."""
        name = name or self._uid('scale')
        (y,) = self._emit('scale', name, [x], [(f'{name}_out', x.shape, out_precision or x.precision)], ['lhs'],
                          {'scale': float(scale), 'layer_class': 'Scale'})
        return y

    def add(self, a: TensorVar, b: TensorVar, out_precision: QuantIntent, name: Optional[str] = None) -> TensorVar:
        name = name or self._uid('add')
        (y,) = self._emit('add', name, [a, b], [(f'{name}_out', a.shape, out_precision)], ['lhs', 'rhs'],
                          {'layer_class': 'Add', 'source_class': 'Add', 'source_layer': name})
        return y

    def layer_norm(self, x: TensorVar, gamma, beta, out_precision: QuantIntent, epsilon: Optional[float] = None,
                   eps_q0: Optional[int] = None, name: Optional[str] = None) -> TensorVar:
        name = name or self._uid('layer_norm')
        g = self.param(f'{name}_gamma', gamma, None)
        b = self.param(f'{name}_beta', beta, None)
        meta = {'layer_class': 'LayerNormalization', 'source_class': 'LayerNormalization', 'source_layer': name,
                'axis': len(x.shape) - 1}
        if epsilon is not None:
            meta['epsilon'] = float(epsilon)
        if eps_q0 is not None:
            meta['eps_q0'] = int(eps_q0)
        (y,) = self._emit('layer_norm', name, [x, g, b], [(f'{name}_out', x.shape, out_precision)],
                          ['lhs', 'gamma', 'beta'], meta)
        return y

    def softmax(self, x: TensorVar, out_precision: QuantIntent, name: Optional[str] = None,
                directives: Optional[Dict] = None) -> TensorVar:
        name = name or self._uid('softmax')
        (y,) = self._emit('softmax', name, [x], [(f'{name}_out', x.shape, out_precision)], ['lhs'],
                          {'axis': len(x.shape) - 1, 'layer_class': 'Softmax', 'source_class': 'Softmax',
                           'source_layer': name}, directives)
        return y

    def build(self):
        from ..model import GPUModel

        self.graph.verify()
        return GPUModel.from_context(self.ctx)
