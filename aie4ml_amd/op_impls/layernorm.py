"""GPU variant of the integer LayerNorm (_LayerNormVariantBase.resolve, src/aie4ml/op_impls/families/
layernorm/layer_norm.py:40-175; parameter packing from layernorm/common.py:36-93)."""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict

import numpy as np

from ..aie_types import AIEDataType, is_float_intent
from ..ir import input_tensor_for_role
from .base import FamilyResolver, OpImplVariant, family_resolver, is_gpu, register_variant
from .precision import aie_rounding_token, resolve_exact_storage_dtype, to_quant_intent, view_shape

# gamma multiplies the Q15 reciprocal standard deviation and is shifted right by GAMMA_SHIFT = 7, so it
# is stored with 7 fractional bits; beta joins the Q15 accumulator before the final shift, so Q15.
GAMMA_FRAC_BITS = 7
BETA_FRAC_BITS = 15


@dataclass(frozen=True)
class LayerNormConfig:
    precision: Dict[str, Any]
    rows: int
    cols: int
    gamma_shift: int
    out_shift: int
    eps_q0: int
    rounding_mode: str
    power_of_two_cols: bool

    def __hash__(self):
        return id(self)


def resolve_eps_q0(node_name: str, metadata: dict, input_frac: int) -> int:
    """epsilon in units of the squared input LSB; must be a positive integer."""
    if 'epsilon' in metadata:
        epsilon = float(metadata['epsilon'])
        if epsilon < 0.0:
            raise ValueError(f'{node_name}: LayerNormalization epsilon must be non-negative, got {epsilon}.')
        exact = epsilon * float(1 << (2 * int(input_frac)))
        eps_q0 = int(round(exact))
        if not math.isclose(exact, float(eps_q0), rel_tol=0.0, abs_tol=1e-6):
            raise ValueError(f'{node_name}: epsilon={epsilon} is not exactly representable as integer EPS_Q0 '
                             f'for input frac={input_frac} (epsilon / input_scale^2 = {exact}).')
        if eps_q0 < 1:
            raise ValueError(f'{node_name}: epsilon={epsilon} maps to EPS_Q0={eps_q0}; '
                             'integer LayerNorm requires a positive variance floor.')
        return eps_q0
    eps_q0 = int(metadata.get('eps_q0', 1))
    if eps_q0 < 1:
        raise ValueError(f'{node_name}: eps_q0 must be positive, got {eps_q0}.')
    return eps_q0


def pack_layernorm_param(values, *, name: str, full_inner: int, frac: int) -> np.ndarray:
    """rint(v * 2^frac) as int16, range-checked (no silent clipping)."""
    arr = np.asarray(values, dtype=np.float64).reshape(-1)
    if int(arr.shape[0]) != int(full_inner):
        raise ValueError(f'LayerNorm parameter {name!r} length {arr.shape[0]} does not match full_inner={int(full_inner)}.')
    if not np.all(np.isfinite(arr)):
        raise ValueError(f'LayerNorm parameter {name!r} contains non-finite values.')
    scale = float(1 << int(frac)) if frac > 0 else 1.0
    scaled = np.rint(arr * scale).astype(np.int64)
    if np.any((scaled < -32768) | (scaled > 32767)):
        raise ValueError(f'LayerNorm parameter {name!r} cannot be represented as signed int16 Q{int(frac)}: '
                         f'value range [{float(arr.min())}, {float(arr.max())}], representable range '
                         f'[{-32768 / scale}, {32767 / scale}].')
    return scaled.astype(np.int16)


@family_resolver('layer_norm')
class LayerNormFamilyResolver(FamilyResolver):
    op_type = 'layer_norm'

    def validate_structure(self, node, _device) -> None:
        x = input_tensor_for_role(node, 'lhs')
        shape = view_shape(node, x, 'inputs')
        if len(shape) < 2:
            raise ValueError(f'{node.name}: LayerNorm requires rank>=2 tensors, got {len(shape)}.')
        axis = int(node.metadata.get('axis', -1))
        axis = axis + len(shape) if axis < 0 else axis
        if axis != len(shape) - 1:
            raise ValueError(f'{node.name}: only last-axis LayerNorm is supported; got axis={axis}.')
        for role in ('gamma', 'beta'):
            if not input_tensor_for_role(node, role).is_parameter:
                raise ValueError(f'{node.name}: LayerNorm {role} must be a constant parameter.')


@register_variant
class LayerNormGpuVariant(OpImplVariant):
    variant_id = 'layer_norm.i8.gfx950.v1'
    op_type = 'layer_norm'
    plevel = 10

    def matches(self, node, device) -> bool:
        if not is_gpu(device):
            return False
        x = input_tensor_for_role(node, 'lhs')
        if x.precision is None or node.outputs[0].precision is None or is_float_intent(x.precision):
            return False
        i = resolve_exact_storage_dtype(x.precision, namespace='lhs', layer_name=node.name)
        o = resolve_exact_storage_dtype(node.outputs[0].precision, namespace='output', layer_name=node.name)
        return i.width == 8 and i.signed and o.width == 8 and o.signed

    def resolve(self, node, _device, _directives=None) -> LayerNormConfig:
        x, out = input_tensor_for_role(node, 'lhs'), node.outputs[0]
        precision = {
            'lhs': resolve_exact_storage_dtype(x.precision, namespace='lhs', layer_name=node.name),
            'output': resolve_exact_storage_dtype(out.precision, namespace='output', layer_name=node.name),
            'gamma': AIEDataType(format='int16', frac=GAMMA_FRAC_BITS),
            'beta': AIEDataType(format='int16', frac=BETA_FRAC_BITS),
        }
        shape = [int(v) for v in view_shape(node, x, 'inputs')]
        cols = shape[-1]
        rows = int(np.prod(shape[:-1], dtype=np.int64))
        return LayerNormConfig(
            precision=precision, rows=rows, cols=cols, gamma_shift=GAMMA_FRAC_BITS,
            out_shift=int(to_quant_intent(out.precision).frac),
            eps_q0=resolve_eps_q0(node.name, node.metadata, int(precision['lhs'].frac)),
            rounding_mode=aie_rounding_token(precision['output']),
            power_of_two_cols=cols > 0 and (cols & (cols - 1)) == 0,
        )

    def validate_config(self, node, config: LayerNormConfig, _device) -> None:
        # the reference additionally requires a power-of-two column count (layer_norm.py:169-170); the GPU
        # kernel divides exactly instead, which is the same arithmetic whenever cols is 2^k
        if not 0 <= config.out_shift <= 15:
            raise ValueError(f'{node.name}: out_shift={config.out_shift} must be in [0, 15]; '
                             'integer LayerNorm cannot left-shift or exceed NORM_SHIFT=15.')
        if config.cols < 1 or config.cols > 65536:
            raise ValueError(f'{node.name}: LayerNorm width {config.cols} outside [1, 65536].')

    def pack(self, inst) -> Dict[str, Any]:
        import torch

        cfg = inst.config
        g = pack_layernorm_param(input_tensor_for_role(inst.node, 'gamma').data, name='gamma', full_inner=cfg.cols,
                                 frac=GAMMA_FRAC_BITS)
        b = pack_layernorm_param(input_tensor_for_role(inst.node, 'beta').data, name='beta', full_inner=cfg.cols,
                                 frac=BETA_FRAC_BITS)
        return {'packed_gamma': torch.from_numpy(g).cuda(), 'packed_beta': torch.from_numpy(b).cuda(),
                'gamma_int': g, 'beta_int': b}

    def get_artifacts(self, inst):
        return [{'name': 'gamma', 'array': inst.artifacts.get('gamma_int')},
                {'name': 'beta', 'array': inst.artifacts.get('beta_int')}]

    def run(self, inst, inputs):
        from .. import ops

        cfg, node = inst.config, inst.node
        x = inputs[input_tensor_for_role(node, 'lhs').name]
        y = ops.layernorm(x, inst.artifacts['packed_gamma'], inst.artifacts['packed_beta'], cfg.out_shift,
                          cfg.rounding_mode, eps_q0=cfg.eps_q0, gamma_shift=cfg.gamma_shift)
        return {node.outputs[0].name: y}
