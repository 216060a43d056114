"""hls4ml model graph -> operator graph, by attribute access only (hls4ml itself is not imported).

Restates the reference's lowering pass (LowerToAieIr, src/aie4ml/frontends/hls4ml/lower.py:29-250) and its helpers
(frontends/hls4ml/utils.py:17-187: the precision bridge, the recovery of a Dense output precision after hls4ml
removed a trailing linear activation, the weight / bias parameter tensors) on the interface an hls4ml ``ModelGraph``
offers: ``get_layers()``, ``get_input_variables()``, ``get_output_variables()``, ``output_vars``, ``config`` and,
per layer, ``name``, ``class_name``, ``inputs``, ``weights``, ``get_attr()``. Node kinds, input roles and metadata are
the ones the reference emits, so the fold / fuse / resolve passes see the same graph. AIE-physical layer
directives (placement, microtiling, parallelism, layout, io_route) have no meaning on the GPU and are not read.
"""

from __future__ import annotations

from typing import Any, Dict, Optional

import numpy as np

from ..aie_types import QuantIntent, RoundingMode, SaturationMode
from ..ir import BackendContext, OpNode, TensorVar, set_input_roles


def _to_quant_intent(precision) -> QuantIntent:
    """hls4ml FixedPrecisionType -> QuantIntent (frontends/hls4ml/utils.py:17-24)."""
    return QuantIntent(width=int(precision.width), frac=int(precision.fractional), signed=bool(precision.signed),
                       rounding=RoundingMode[precision.rounding_mode.name],
                       saturation=SaturationMode[precision.saturation_mode.name])


def _precision_of(var) -> Optional[QuantIntent]:
    precision = getattr(getattr(var, 'type', None), 'precision', None)
    if precision is None:
        return None
    try:
        return _to_quant_intent(precision)
    except Exception:  # noqa: BLE001  (an unknown precision type leaves the tensor without an intent, as in the reference)
        return None


def _assert_true_pointwise(layer) -> None:
    """passes/utils.py:30-62."""
    g = layer.get_attr
    if layer.class_name == 'Conv1D':
        if not (g('filt_width') == 1 and g('stride_width') == 1 and g('pad_left') == 0 and g('pad_right') == 0
                and g('in_width') == g('out_width')):
            raise ValueError(f'{layer.name}: PointwiseConv1D is not true pointwise.')
        return
    if not ((g('filt_height'), g('filt_width')) == (1, 1) and (g('stride_height'), g('stride_width')) == (1, 1)
            and (g('pad_top'), g('pad_bottom'), g('pad_left'), g('pad_right')) == (0, 0, 0, 0)
            and (g('in_height'), g('in_width')) == (g('out_height'), g('out_width'))):
        raise ValueError(f'{layer.name}: PointwiseConv2D is not true pointwise.')


def is_pointwise_dense(layer) -> bool:
    if layer.class_name not in ('Conv1D', 'Conv2D'):
        return False
    _assert_true_pointwise(layer)
    return True


def _post_activation_precision(layer, model) -> Optional[QuantIntent]:
    """The precision a removed trailing linear activation would have given the Dense output
    (frontends/hls4ml/utils.py:37-68)."""
    config = model.config
    lnp = getattr(config, 'layer_name_precision', {}) or {}
    linear_key = f'{layer.name.lower()}_linear_result'
    if linear_key not in lnp:
        return None
    existing = {lr.name.lower() for lr in model.get_layers()}
    keys = list(lnp.keys())
    for key in keys[keys.index(linear_key) + 1:]:
        if not key.endswith('_result'):
            continue
        val = lnp[key]
        if val == 'auto':
            continue
        if key[:-len('_result')] in existing:
            return None
        try:
            return _to_quant_intent(config.backend.convert_precision_string(val))
        except Exception:  # noqa: BLE001
            return None
    return None


def _weight_tensors(layer, graph):
    """Weight and bias parameter tensors of a Dense / pointwise Conv layer (frontends/hls4ml/utils.py:127-187)."""
    weight_var = layer.weights.get('weight')
    if weight_var is None:
        raise RuntimeError(f'Layer {layer.name}: Dense node has no weight variable.')
    weight_precision = getattr(weight_var.type, 'precision', None)
    if weight_precision is None:
        raise RuntimeError(f'Layer {layer.name}: weight has no precision metadata.')
    pre_quantized = layer.get_attr('weight_quantizer') is not None
    raw = _to_quant_intent(weight_precision)
    if pre_quantized:
        weight_data, weight_intent = weight_var.data, raw
    else:  # raw floats (a Dense that hls4ml turned into a pointwise convolution): round to nearest even when packing
        weight_data = getattr(weight_var, 'data_unquantized', weight_var.data)
        weight_intent = QuantIntent(width=raw.width, frac=raw.frac, signed=raw.signed, rounding=RoundingMode.RND_CONV,
                                    saturation=raw.saturation)
    weight_data = np.asarray(weight_data, dtype=np.float64)
    weight_tv = TensorVar(name=f'{layer.name}_weight', shape=tuple(weight_data.shape), precision=weight_intent, data=weight_data)
    graph.add_tensor(weight_tv)

    bias_var = layer.weights.get('bias')
    if bias_var is None or bias_var.data is None:
        return weight_tv, None
    bias_precision = getattr(bias_var.type, 'precision', None)
    if bias_precision is None:
        raise RuntimeError(f'Layer {layer.name}: bias has no precision metadata.')
    bias_intent = _to_quant_intent(bias_precision)
    if pre_quantized:
        bias_data = np.asarray(bias_var.data, dtype=np.float64)
    else:
        delta = 1.0 / (1 << bias_intent.frac)
        bias_data = np.round(np.asarray(getattr(bias_var, 'data_unquantized', bias_var.data), dtype=np.float64) / delta) * delta
    bias_tv = TensorVar(name=f'{layer.name}_bias', shape=tuple(bias_data.shape), precision=bias_intent, data=bias_data)
    graph.add_tensor(bias_tv)
    return weight_tv, bias_tv


def _map_op_type(layer) -> str:
    if layer.class_name == 'Dense' or is_pointwise_dense(layer):
        return 'dense'
    if layer.class_name == 'Transpose':
        return 'transpose'
    if layer.class_name == 'LayerNormalization':
        return 'layer_norm'
    return layer.class_name.lower()


def _collect_metadata(layer, node: OpNode) -> None:
    meta: Dict[str, Any] = {}
    if layer.class_name == 'Dense' or is_pointwise_dense(layer):
        n_in = layer.get_attr('n_in') if layer.class_name == 'Dense' else layer.get_attr('n_chan')
        n_out = layer.get_attr('n_out') if layer.class_name == 'Dense' else layer.get_attr('n_filt')
        if n_in is None or n_out is None:
            raise ValueError(f'{layer.name}: missing n_in/n_out for {layer.class_name}.')
        meta.update(n_in=int(n_in), n_out=int(n_out), use_bias=layer.get_attr('bias_data') is not None)
        meta['input_roles'] = ['lhs', 'rhs'] + (['bias'] if meta['use_bias'] else [])
    if layer.class_name == 'ApplyAlpha':
        scale = layer.get_attr('scale_data')
        if scale is not None:
            meta['scale'] = np.asarray(scale, dtype=np.float64).flatten().tolist()
    if layer.class_name == 'LayerNormalization':
        meta['input_roles'] = ['lhs', 'gamma', 'beta']
        if layer.get_attr('epsilon') is not None:
            meta['epsilon'] = float(layer.get_attr('epsilon'))
    if layer.class_name == 'Activation':
        meta['input_roles'] = ['lhs']
        act = (layer.get_attr('activation', '') or '').lower()
        if act:
            meta['activation'] = act
    if layer.class_name == 'Transpose':
        meta['input_roles'] = ['lhs']
        perm = layer.get_attr('perm')
        if perm is None:
            raise ValueError(f'{layer.name}: missing Transpose perm attribute.')
        meta['perm'] = [int(x) for x in perm]
        meta['data_format'] = layer.get_attr('data_format')
    meta['layer_class'] = layer.class_name
    if is_pointwise_dense(layer):
        meta['source_class'] = layer.class_name
        meta['layer_class'] = 'Dense'
    meta['source_layer'] = layer.name
    node.metadata.update(meta)


def lower_hls4ml_model(model, config: Optional[Dict[str, Any]] = None) -> BackendContext:
    """Build the operator graph of an hls4ml model. `config` overrides / supplies the run configuration the
    reference reads from the model's AIEConfig block (BatchSize, Iterations, ComputeDtype)."""
    aie_cfg = {}
    get_value = getattr(getattr(model, 'config', None), 'get_config_value', None)
    if get_value is not None:
        aie_cfg = dict(get_value('AIEConfig', {}) or {})
    aie_cfg.update(config or {})
    if 'BatchSize' not in aie_cfg:
        raise KeyError("hls4ml lowering needs a BatchSize (model AIEConfig or the config argument).")
    batch_size = int(aie_cfg['BatchSize'])
    frontend_policy = (get_value('AIEFrontendPolicy', {}) or {}) if get_value is not None else {}
    batch_included = bool(frontend_policy.get('TensorsHaveBatch', False))
    ctx = BackendContext(config=aie_cfg)
    graph = ctx.ir.logical

    def canon(shape):
        dims = tuple(int(x) for x in shape)
        return dims if batch_included else (batch_size,) + dims

    layers = list(model.get_layers())
    input_var = model.get_input_variables()[0]
    if input_var.name not in graph.tensors:
        # the reference keeps the input variable's own shape here and relies on its buffer compaction for the batch
        # axis; the GPU executor wants every activation with its batch axis, so the input is canonicalised as well
        graph.add_tensor(TensorVar(name=input_var.name, shape=canon(input_var.shape), precision=_precision_of(input_var)))
    graph.mark_graph_input(input_var.name)

    for layer in layers:
        var = model.output_vars[layer.name]
        if var.name in graph.tensors:
            continue
        prec = _precision_of(var)
        if layer.class_name == 'Dense' or is_pointwise_dense(layer):
            override = _post_activation_precision(layer, model)
            if override is not None:
                prec = override
        graph.add_tensor(TensorVar(name=var.name, shape=canon(var.shape), precision=prec))

    node_map: Dict[str, OpNode] = {}
    params: Dict[str, tuple] = {}
    for layer in layers:
        node = OpNode(name=f'{layer.name}_aie', op_type=_map_op_type(layer))
        if layer.class_name.lower() == 'input':
            node.is_placeholder = True
        _collect_metadata(layer, node)
        if node.op_type == 'dense':
            params[layer.name] = _weight_tensors(layer, graph)
        if node.op_type == 'layer_norm':
            pair = []
            for weight_name, role in (('scale', 'gamma'), ('bias', 'beta')):
                wvar = layer.weights.get(weight_name)
                if wvar is None:
                    raise RuntimeError(f'{layer.name}: LayerNormalization missing {weight_name!r} weight.')
                data = np.asarray(wvar.data, dtype=np.float64)
                tv = TensorVar(name=f'{layer.name}_{role}', shape=tuple(data.shape), precision=_precision_of(wvar), data=data)
                graph.add_tensor(tv)
                pair.append(tv)
            params[layer.name] = tuple(pair)
        tv = graph.tensors[model.output_vars[layer.name].name]
        tv.producer = node
        node.outputs.append(tv)
        if node.op_type == 'transpose':
            perm = node.metadata.get('perm')
            if len(perm) == len(tv.shape) - 1:  # hls4ml permutations leave out the batch axis
                node.metadata['perm'] = [0] + [int(p) + 1 for p in perm]
        graph.add_node(node)
        node_map[layer.name] = node

    for layer in layers:
        node = node_map[layer.name]
        if layer.class_name.lower() == 'input':
            continue
        for src in layer.inputs:
            var = input_var if src == 'input' else model.output_vars[src]
            tv = graph.tensors[var.name]
            node.inputs.append(tv)
            tv.consumers.append(node)
        if layer.name in params:
            first, second = params[layer.name]
            node.inputs.append(first)
            first.consumers.append(node)
            if second is not None:
                node.inputs.append(second)
                second.consumers.append(node)
        roles = list(node.metadata.get('input_roles') or [])
        if roles:
            set_input_roles(node, node.inputs, roles)
        elif len(node.inputs) == 2:  # Merge-style layers carry no role list: left and right operand in input order
            set_input_roles(node, node.inputs, ['lhs', 'rhs'])
        elif len(node.inputs) == 1:
            set_input_roles(node, node.inputs, ['lhs'])

    for out_var in model.get_output_variables():
        graph.mark_graph_output(out_var.name)
    return ctx


def from_hls4ml(model, config: Optional[Dict[str, Any]] = None):
    """hls4ml ModelGraph -> GPUModel (the counterpart of AIEModel.from_hls4ml, src/aie4ml/model.py:156-162)."""
    from ..model import GPUModel

    return GPUModel.from_context(lower_hls4ml_model(model, config), source_model=model)
