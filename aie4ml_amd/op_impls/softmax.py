"""GPU variants of the integer Softmax: accurate integer exp (the default) and the HCCS surrogate.

Selection and constants follow src/aie4ml/op_impls/families/softmax/softmax.py:27-349 and
softmax/common.py:59-108; structural rules follow softmax/resolver.py:13-25.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Any, ClassVar, Dict

import numpy as np

from ..aie_types import is_float_intent
from ..ir import input_tensor_for_role
from .base import FamilyResolver, OpImplVariant, family_resolver, is_gpu, register_variant
from .precision import resolve_exact_storage_dtype, view_shape

DEFAULT_INV_SHIFT = 15
EXP_ZF = 8                    # fractional bits of the base-2 exponent in the integer exp
EXP_KQ_MAX = 32767 // 255     # (max - x) * EXP_KQ must fit int16 for the largest int8 gap


@dataclass(frozen=True)
class SoftmaxConfig:
    precision: Dict[str, Any]
    rows: int
    cols: int
    param_sets: int
    inv_shift: int
    use_clb: bool
    hccs: Dict[str, Any] = field(default_factory=dict)
    approximation: str = 'hccs'
    exp_kq: int = 0
    rounding_mode: str = 'floor'  # hard-wired in the reference's kernel parameters

    def __hash__(self):
        return id(self)


def requested_approximation(node) -> str:
    """No `approximation` directive -> the accurate integer exp, which needs no calibration."""
    approx = (node.directives or {}).get('approximation')
    return 'exp' if approx is None else str(approx).lower()


def exp_kq(input_scale: float) -> int:
    """log2(e) * input_scale in Q8: the base-2 exponent step per unit logit gap."""
    return int(round(math.log2(math.e) * float(input_scale) * (1 << EXP_ZF)))


def _int_array(value, *, name: str, lo: int, hi: int) -> np.ndarray:
    arr = np.asarray(value, dtype=np.int64).reshape(-1)
    if arr.size == 0:
        raise ValueError(f'HCCS Softmax parameter {name!r} must not be empty.')
    if np.any((arr < lo) | (arr > hi)):
        raise ValueError(f'HCCS Softmax parameter {name!r} must be in [{lo}, {hi}].')
    return arr


def infer_hccs_param_sets(hccs: Dict[str, Any]) -> int:
    lengths = [int(np.asarray(hccs[k]).reshape(-1).size) for k in ('B', 'S', 'Dmax')]
    if any(n < 1 for n in lengths):
        raise ValueError('HCCS Softmax parameters must not be empty.')
    multi = [n for n in lengths if n > 1]
    inferred = multi[0] if multi else 1
    if any(n != inferred for n in multi):
        raise ValueError(f'HCCS Softmax non-scalar parameter lengths must match, got {multi}.')
    explicit = hccs.get('param_sets')
    sets = int(explicit) if explicit is not None else inferred
    if sets < 1:
        raise ValueError(f'HCCS Softmax param_sets must be positive, got {sets}.')
    if inferred > 1 and sets != inferred:
        raise ValueError(f'HCCS Softmax param_sets={sets} must match non-scalar parameter length {inferred}.')
    return sets


def validate_hccs_params(hccs: Dict[str, Any], *, cols: int, param_sets: int) -> None:
    """Calibration constants against the kernel's fixed-point ranges."""
    if int(param_sets) != 1:
        raise ValueError(f'HCCS Softmax compile-time scalar parameter packing requires param_sets=1, got {param_sets}.')
    b = _int_array(hccs['B'], name='B', lo=0, hi=32767)
    s = _int_array(hccs['S'], name='S', lo=0, hi=127)
    d = _int_array(hccs['Dmax'], name='Dmax', lo=0, hi=127)
    floor_score = int(b[0]) - int(s[0]) * int(d[0])
    if floor_score < 0:
        raise ValueError(f'HCCS Softmax requires B - S*Dmax >= 0 for every row; row 0 gives {floor_score}.')
    if floor_score * int(cols) < 256:
        raise ValueError('HCCS Softmax requires cols * (B - S*Dmax) >= 256 for reciprocal range; '
                         f'row 0 gives {floor_score * int(cols)}.')
    if int(b[0]) * int(cols) > 32767:
        raise ValueError('HCCS Softmax requires cols * B <= 32767 so score sum fits int16 range.')


@family_resolver('softmax')
class SoftmaxFamilyResolver(FamilyResolver):
    op_type = 'softmax'

    def validate_structure(self, node, _device) -> None:
        x, out = input_tensor_for_role(node, 'lhs'), node.outputs[0]
        ishape = tuple(int(v) for v in view_shape(node, x, 'inputs'))
        oshape = tuple(int(v) for v in view_shape(node, out, 'outputs'))
        if len(ishape) < 2:
            raise ValueError(f'{node.name}: Softmax requires rank>=2 tensors, got {len(ishape)}.')
        if ishape != oshape:
            raise ValueError(f'{node.name}: Softmax input/output shapes must match, got {ishape} and {oshape}.')
        axis = int(node.metadata.get('axis', -1))
        axis = axis + len(ishape) if axis < 0 else axis
        if axis != len(ishape) - 1:
            raise ValueError(f'{node.name}: only last-axis Softmax is supported; got axis={axis}.')


class _SoftmaxGpuBase(OpImplVariant):
    approximation: ClassVar[str]
    op_type = 'softmax'
    plevel = 10

    def matches(self, node, device) -> bool:
        if not is_gpu(device) or requested_approximation(node) != self.approximation:
            return False
        x = input_tensor_for_role(node, 'lhs')
        if x.precision is None or is_float_intent(x.precision):
            return False
        return resolve_exact_storage_dtype(x.precision, namespace='lhs', layer_name=node.name).format == 'int8'

    def _resolve_params(self, node, directives, cols: int) -> Dict[str, Any]:
        raise NotImplementedError

    def resolve(self, node, _device, directives=None) -> SoftmaxConfig:
        x, out = input_tensor_for_role(node, 'lhs'), node.outputs[0]
        if out.precision is None:
            raise ValueError(f'{node.name}: missing precision metadata for softmax.')
        precision = {
            'lhs': resolve_exact_storage_dtype(x.precision, namespace='lhs', layer_name=node.name),
            'output': resolve_exact_storage_dtype(out.precision, namespace='output', layer_name=node.name),
        }
        shape = [int(v) for v in view_shape(node, x, 'inputs')]
        params = self._resolve_params(node, directives if directives is not None else node.directives, shape[-1])
        return SoftmaxConfig(precision=precision, rows=int(np.prod(shape[:-1], dtype=np.int64)), cols=shape[-1],
                             approximation=self.approximation, **params)

    def validate_config(self, node, config: SoftmaxConfig, _device) -> None:
        fmt = config.precision['output'].format
        if fmt not in ('uint8', 'int16'):
            raise ValueError(f'{node.name}: {self.variant_id} requires uint8 or int16 output, got {fmt!r}.')
        if config.cols < 1 or config.cols > 65536:
            raise ValueError(f'{node.name}: softmax axis length {config.cols} outside [1, 65536].')


@register_variant
class SoftmaxExpGpuVariant(_SoftmaxGpuBase):
    """Accurate integer Softmax (2nd-order integer exp) — what a plain Softmax lowers to."""

    variant_id = 'softmax.exp.i8.gfx950.v1'
    approximation = 'exp'

    def _resolve_params(self, node, _directives, _cols):
        x = input_tensor_for_role(node, 'lhs')
        frac = resolve_exact_storage_dtype(x.precision, namespace='lhs', layer_name=node.name).frac
        temperature = float(node.trait_data('input_scale').get('scale', 1.0))
        return {'param_sets': 1, 'inv_shift': DEFAULT_INV_SHIFT, 'use_clb': False, 'hccs': {},
                'exp_kq': exp_kq((2.0 ** -int(frac)) * temperature)}

    def validate_config(self, node, config, device) -> None:
        super().validate_config(node, config, device)
        if not 1 <= int(config.exp_kq) <= EXP_KQ_MAX:
            scale = float(node.trait_data('input_scale').get('scale', 1.0))
            raise ValueError(f'{node.name}: exp Softmax needs 1 <= EXP_KQ <= {EXP_KQ_MAX}, got {config.exp_kq} for '
                             f'input_scale={scale}. The input fixed-point scale is out of range (roughly frac in '
                             '[2, 9]): too fine and every logit gap rounds to zero (uniform output); too coarse and '
                             '(max-x)*KQ overflows int16. Requantise the softmax input.')

    def run(self, inst, inputs):
        from .. import ops

        cfg, node = inst.config, inst.node
        x = inputs[input_tensor_for_role(node, 'lhs').name]
        y = ops.softmax_exp(x, cfg.exp_kq, cfg.inv_shift, out_kind=cfg.precision['output'].format)
        return {node.outputs[0].name: y}


@register_variant
class SoftmaxHccsGpuVariant(_SoftmaxGpuBase):
    """Head-calibrated clipped-linear surrogate: score = B - S*min(max-x, Dmax). Not a drop-in for a
    float Softmax; needs the `hccs: {B, S, Dmax}` calibration directive."""

    variant_id = 'softmax.hccs.i8.gfx950.v1'
    approximation = 'hccs'

    def _resolve_params(self, node, directives, _cols):
        hccs = dict((directives or {}).get('hccs', {}) or {})
        missing = [k for k in ('B', 'S', 'Dmax') if k not in hccs]
        if missing:
            raise ValueError(f'{node.name}: HCCS Softmax directives missing {", ".join(missing)}.')
        scale = float(node.trait_data('input_scale').get('scale', 1.0))
        if abs(scale - 1.0) > 1e-9:
            raise ValueError(f'{node.name}: {self.variant_id} cannot apply a runtime input_scale={scale}; bake the '
                             'softmax temperature into the HCCS B/S/Dmax calibration, or drop the approximation '
                             'directive to use the accurate exp Softmax, which applies input_scale directly.')
        return {'param_sets': int(infer_hccs_param_sets(hccs)), 'inv_shift': int(hccs.get('inv_shift', DEFAULT_INV_SHIFT)),
                'use_clb': bool(hccs.get('use_clb', False)), 'hccs': hccs, 'exp_kq': 0}

    def validate_config(self, node, config, device) -> None:
        super().validate_config(node, config, device)
        if config.param_sets != 1:
            raise ValueError(f'{node.name}: {self.variant_id} does not support multi-head param_sets='
                             f'{config.param_sets}; lower attention to one Softmax op per head.')
        if not 1 <= int(config.inv_shift) <= 30:
            raise ValueError(f'{node.name}: HCCS Softmax inv_shift must be in [1, 30], got {config.inv_shift}.')
        if int(config.inv_shift) > 23:
            raise NotImplementedError(f'{node.name}: inv_shift={config.inv_shift} overflows the 32-bit reciprocal '
                                      'numerator 255 << inv_shift; the GPU kernel accepts [1, 23].')
        validate_hccs_params(config.hccs, cols=config.cols, param_sets=config.param_sets)

    def run(self, inst, inputs):
        from .. import ops

        cfg, node = inst.config, inst.node
        x = inputs[input_tensor_for_role(node, 'lhs').name]
        h = cfg.hccs
        y = ops.softmax_hccs(x, int(np.asarray(h['B']).reshape(-1)[0]), int(np.asarray(h['S']).reshape(-1)[0]),
                             int(np.asarray(h['Dmax']).reshape(-1)[0]), cfg.inv_shift, cfg.use_clb,
                             out_kind=cfg.precision['output'].format)
        return {node.outputs[0].name: y}
