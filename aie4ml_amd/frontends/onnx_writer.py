"""Builds ONNX Q/DQ models (onnx_proto.Model) in the form quantisation-aware exporters produce: float graph
inputs, integer initializers behind DequantizeLinear, a QuantizeLinear / DequantizeLinear pair after every
operator. Used to write the synthetic models of the benchmark configurations to .onnx files that both this
importer and the reference's `from_onnx` accept."""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np

from ..aie_types import QuantIntent
from ..quant_utils import dtype_for_precision
from . import onnx_proto as op


class QdqWriter:
    def __init__(self, name: str = 'graph', opset: int = 17):
        self.model = op.Model(graph=op.Graph(name=name), opset={'': opset}, producer_name='aie4ml_amd')
        self._names: Dict[str, int] = {}

    def _unique(self, base: str) -> str:
        n = self._names.get(base, 0)
        self._names[base] = n + 1
        return base if n == 0 else f'{base}_{n}'

    def const(self, name: str, array) -> str:
        name = self._unique(name)
        self.model.graph.initializers.append(op.Tensor(name, np.asarray(array)))
        return name

    def node(self, op_type: str, inputs: Sequence[str], n_out: int = 1, name: Optional[str] = None, **attrs) -> List[str]:
        name = self._unique(name or op_type.lower())
        outs = [f'{name}_out{i}' if n_out > 1 else f'{name}_out' for i in range(n_out)]
        self.model.graph.nodes.append(op.Node(op_type, list(inputs), outs, name, dict(attrs)))
        return outs

    def _qparams(self, base: str, intent: QuantIntent):
        dt = dtype_for_precision(intent.width, intent.signed)
        return self.const(f'{base}_scale', np.array(2.0 ** -intent.frac, dtype=np.float32)), self.const(f'{base}_zp', np.zeros((), dtype=dt))

    def qdq(self, value: str, intent: QuantIntent, name: Optional[str] = None) -> str:
        """QuantizeLinear + DequantizeLinear: declares `value` to be stored with `intent`."""
        base = name or f'{value}_q'
        scale, zp = self._qparams(base, intent)
        (q,) = self.node('QuantizeLinear', [value, scale, zp], name=f'{base}_quant')
        (d,) = self.node('DequantizeLinear', [q, scale, zp], name=f'{base}_dequant')
        return d

    def input(self, name: str, shape: Sequence[int], intent: QuantIntent) -> str:
        self.model.graph.inputs.append(op.ValueInfo(name, op.FLOAT, tuple(int(s) for s in shape)))
        return self.qdq(name, intent, name=f'{name}_q')

    def weight(self, name: str, values, intent: QuantIntent) -> str:
        """An integer initializer (values must lie on the intent's grid) behind a DequantizeLinear."""
        scaled = np.asarray(values, dtype=np.float64) * 2.0 ** intent.frac
        ints = np.rint(scaled)
        if not np.array_equal(ints, scaled):
            raise ValueError(f'{name}: values are not on the 2^-{intent.frac} grid')
        dt = dtype_for_precision(intent.width, intent.signed)
        info = np.iinfo(dt)
        if ints.min() < info.min or ints.max() > info.max:
            raise ValueError(f'{name}: values do not fit {np.dtype(dt).name}')
        raw = self.const(name, ints.astype(dt))
        scale, zp = self._qparams(name, intent)
        (d,) = self.node('DequantizeLinear', [raw, scale, zp], name=f'{name}_dequant')
        return d

    def output(self, value: str, shape: Sequence[int]) -> None:
        self.model.graph.outputs.append(op.ValueInfo(value, op.FLOAT, tuple(int(s) for s in shape)))

    def to_bytes(self) -> bytes:
        return op.serialize_model(self.model)
