"""Stand-ins for the hls4ml objects the lowering reads (hls4ml is not installed here): just the attributes and
methods of ModelGraph / Layer / Variable / FixedPrecisionType that src/aie4ml/frontends/hls4ml/lower.py and
utils.py touch. Built the way hls4ml builds a QKeras MLP: an Input layer, Dense layers with pre-quantised weights
(weight_quantizer set), Activation layers (relu / linear), optionally ApplyAlpha."""

from enum import Enum
from types import SimpleNamespace

import numpy as np


class RoundingMode(Enum):
    TRN = 1
    RND = 2
    RND_CONV = 3


class SaturationMode(Enum):
    WRAP = 1
    SAT = 2


def fixed(width, integer, signed=True, rounding='TRN', saturation='WRAP'):
    return SimpleNamespace(width=width, integer=integer, fractional=width - integer, signed=signed,
                           rounding_mode=RoundingMode[rounding], saturation_mode=SaturationMode[saturation])


def variable(name, shape, precision, data=None):
    return SimpleNamespace(name=name, shape=tuple(shape), type=SimpleNamespace(precision=precision), data=data)


class Layer:
    def __init__(self, name, class_name, inputs, attrs=None, weights=None):
        self.name, self.class_name, self.inputs = name, class_name, list(inputs)
        self.attributes = dict(attrs or {})
        self.weights = dict(weights or {})

    def get_attr(self, key, default=None):
        return self.attributes.get(key, default)


class Model:
    """`layers`: Layer objects in execution order; `out_vars`: layer name -> output variable."""

    def __init__(self, layers, out_vars, aie_config, layer_name_precision=None):
        self._layers = list(layers)
        self.output_vars = dict(out_vars)
        values = {'AIEConfig': dict(aie_config)}
        self.config = SimpleNamespace(get_config_value=lambda key, default=None: values.get(key, default),
                                      layer_name_precision=dict(layer_name_precision or {}))

    def get_layers(self):
        return list(self._layers)

    def get_input_variables(self):
        return [self.output_vars[self._layers[0].name]]

    def get_output_variables(self):
        return [self.output_vars[self._layers[-1].name]]


def quantise(values, precision):
    """What hls4ml stores for a pre-quantised weight: values on the 2^-fractional grid (round to nearest, saturate)."""
    scale = 2.0 ** precision.fractional
    lo = -(2 ** (precision.width - 1)) if precision.signed else 0
    hi = 2 ** (precision.width - 1) - 1 if precision.signed else 2 ** precision.width - 1
    return np.clip(np.rint(np.asarray(values) * scale), lo, hi) / scale


def qkeras_mlp(dims, batch, bits=8, int_bits=3, seed=0, relu_last=False, alpha=None):
    """Input -> [Dense(+bias) -> Activation(relu)] ... -> Dense -> Activation(linear), as hls4ml lowers
    tests/test_hls4ml_dense.py's QKeras network. Returns (Model, float weights [(W, b), ...])."""
    r = np.random.default_rng(seed)
    act_t = fixed(bits, int_bits, True, 'RND_CONV', 'SAT')           # quantized_bits(bits, int_bits - 1) activations
    relu_t = fixed(bits, 0, False, 'RND_CONV', 'SAT')                # quantized_relu(bits, 0)
    w_t = fixed(bits, 3, True, 'RND_CONV', 'SAT')                    # quantized_bits(bits, 2, alpha=1) weights
    layers, out_vars, weights = [], {}, []
    x_var = variable('input_layer', (dims[0],), act_t)
    layers.append(Layer('input_layer', 'Input', []))
    out_vars['input_layer'] = x_var
    prev = 'input_layer'
    for i in range(len(dims) - 1):
        last = i == len(dims) - 2
        W = quantise(r.normal(0, 0.6, (dims[i], dims[i + 1])), w_t)
        b = quantise(r.normal(0, 0.3, dims[i + 1]), w_t)
        weights.append((W, b))
        name = f'dense{i}'
        acc_t = fixed(2 * bits + 8, int_bits + 3 + 8, True)          # hls4ml's accumulator-width result type
        layers.append(Layer(name, 'Dense', [prev if prev != 'input_layer' else 'input'],
                            {'n_in': dims[i], 'n_out': dims[i + 1], 'bias_data': b, 'weight_quantizer': object()},
                            {'weight': variable(f'{name}_w', W.shape, w_t, W), 'bias': variable(f'{name}_b', b.shape, w_t, b)}))
        out_vars[name] = variable(f'{name}_out', (dims[i + 1],), acc_t)
        prev = name
        if alpha is not None and i == 0:
            layers.append(Layer(f'alpha{i}', 'ApplyAlpha', [prev], {'scale_data': np.full(dims[i + 1], alpha)}))
            out_vars[f'alpha{i}'] = variable(f'alpha{i}_out', (dims[i + 1],), acc_t)
            prev = f'alpha{i}'
        kind = 'relu' if (not last or relu_last) else 'linear'
        layers.append(Layer(f'act{i}', 'Activation', [prev], {'activation': kind}))
        out_vars[f'act{i}'] = variable(f'act{i}_out', (dims[i + 1],), relu_t if kind == 'relu' else act_t)
        prev = f'act{i}'
    return Model(layers, out_vars, {'BatchSize': batch, 'Iterations': 1}), weights
