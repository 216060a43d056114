"""GPU variants of the matmul family: Dense (static weights, bias, ReLU) and dynamic MatMul.

Numeric resolution follows _DenseVariantBase.resolve / _MatmulVariantBase.resolve
(src/aie4ml/op_impls/families/matmul/dense.py:94-133, matmul.py:47-98) and _resolve_numeric /
_resolve_bias_dtype / _resolve_output_scale_shift (resolver.py:110-175); weight and bias quantisation
follows _quantize_weight_bias (dense.py:135-171). The AIE tiling / cascade / staging search of the
reference has no GPU counterpart and is not reproduced.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

import numpy as np

from ..aie_types import AIEDataType, is_float_intent
from ..ir import input_role, input_tensor_for_role
from ..quant_utils import quantize_to_int
from .base import FamilyResolver, OpImplVariant, family_resolver, is_gpu, register_variant
from .precision import (aie_rounding_token, is_identity, is_last_two_swap, resolve_accumulator_output_shift,
                        resolve_exact_storage_dtype, to_quant_intent, view_perm, view_shape)


@dataclass(frozen=True)
class DenseFlags:
    use_relu: bool
    transpose_lhs: bool
    use_bias: bool


@dataclass(frozen=True)
class MatmulFlags:
    transpose_lhs: bool
    transpose_rhs: bool


@dataclass(frozen=True)
class DenseConfig:
    precision: Dict[str, Any]
    shift: int
    shift_per_channel: Optional[Tuple[int, ...]]  # extension: one right shift per output feature
    accumulator_tag: str
    rounding_mode: str
    flags: DenseFlags
    n_in: int
    n_out: int

    def __hash__(self):
        return id(self)


@dataclass(frozen=True)
class MatmulConfig:
    precision: Dict[str, Any]
    shift: int
    accumulator_tag: str
    rounding_mode: str
    flags: MatmulFlags

    def __hash__(self):
        return id(self)


def _resolve_numeric(node) -> Dict[str, AIEDataType]:
    lhs, rhs, out = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs'), node.outputs[0]
    if any(t.precision is None for t in (lhs, rhs, out)):
        raise ValueError(f'{node.name}: missing precision metadata for {node.op_type}.')
    if any(is_float_intent(t.precision) for t in (lhs, rhs, out)):
        raise NotImplementedError(f'{node.name}: float {node.op_type} has no GPU variant; the integer path is int8.')
    resolved = {
        'lhs': resolve_exact_storage_dtype(lhs.precision, namespace='lhs', layer_name=node.name),
        'rhs': resolve_exact_storage_dtype(rhs.precision, namespace='rhs', layer_name=node.name),
        'output': resolve_exact_storage_dtype(out.precision, namespace='output', layer_name=node.name),
    }
    if resolved['lhs'].width <= 8 and resolved['rhs'].width > 8:
        raise RuntimeError(f'{node.name}: unsupported int8 x int16 precision mix for AIE implementations; '
                           'no implementation variant available.')
    # 8 x 8 and 16 x 8 accumulate in 32 bits, 16 x 16 in 64 (infer_accumulator_tag, precision.py:116-123)
    wide = resolved['lhs'].width > 8 and resolved['rhs'].width > 8
    resolved['acc'] = AIEDataType(format='int64' if wide else 'int32', frac=int(resolved['lhs'].frac + resolved['rhs'].frac))
    return resolved


def _resolve_bias_dtype(node, precision) -> AIEDataType:
    bias = next((t for t in node.inputs if t.is_parameter and input_role(node, t.name) == 'bias'), None)
    frac = int(precision['lhs'].frac) + int(precision['rhs'].frac)
    if bias is not None and bias.precision is not None:
        q = to_quant_intent(bias.precision)
        return AIEDataType(format='int32', frac=frac, rounding=q.rounding, saturation=q.saturation)
    return AIEDataType(format='int32', frac=frac)


def _resolve_output_scale_shift(node) -> int:
    trait = node.traits.get('output_scale')
    if trait is None:
        return 0
    scale = float(trait.data['scale'])
    if scale <= 0.0 or scale > 1.0:
        raise ValueError(f'{node.name}: fused output scale must be in the range (0, 1], got {scale}.')
    shift = int(round(-math.log2(scale)))
    if not math.isclose(scale, math.ldexp(1.0, -shift), rel_tol=0.0, abs_tol=1e-12):
        raise NotImplementedError(f'{node.name}: fused output scale {scale} is not a power of two; '
                                  'fixed-point multiplier scaling is not implemented.')
    return shift


# (lhs, rhs) storage widths (matmul/common.py:52)
_SUPPORTED_INT_WIDTH_COMBOS = frozenset({(8, 8), (16, 8), (16, 16)})


def _bitwidths_supported(node, device) -> bool:
    if not is_gpu(device):
        return False
    lhs, rhs = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
    if is_float_intent(lhs.precision) or is_float_intent(rhs.precision) or lhs.precision is None or rhs.precision is None:
        return False
    lw = resolve_exact_storage_dtype(lhs.precision, namespace='lhs', layer_name=node.name).width
    rw = resolve_exact_storage_dtype(rhs.precision, namespace='rhs', layer_name=node.name).width
    return (lw, rw) in _SUPPORTED_INT_WIDTH_COMBOS


def _check_out_format(node, fmt: str) -> None:
    if fmt not in ('int8', 'uint8', 'int16'):
        raise NotImplementedError(f'{node.name}: GPU {node.op_type} writes int8, uint8 or int16, not {fmt!r}.')


@family_resolver('dense')
class DenseFamilyResolver(FamilyResolver):
    op_type = 'dense'

    def validate_structure(self, node, _device) -> None:
        lhs, rhs = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        if not rhs.is_parameter:
            raise ValueError(f'{node.name}: dense weights must be a parameter tensor.')
        w = np.asarray(rhs.data)
        if w.ndim < 2:
            raise ValueError(f'{node.name}: weight matrix must have at least 2 dimensions, got {w.ndim}.')
        lhs_shape = view_shape(node, lhs, 'inputs')
        if int(lhs_shape[-1]) != int(w.shape[-2]):
            raise ValueError(f'{node.name}: input has {lhs_shape[-1]} features but the weights expect {w.shape[-2]}.')


@family_resolver('matmul')
class MatmulFamilyResolver(FamilyResolver):
    op_type = 'matmul'

    def validate_structure(self, node, _device) -> None:
        lhs, rhs = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        ls, rs = view_shape(node, lhs, 'inputs'), view_shape(node, rhs, 'inputs')
        if len(ls) < 2 or len(rs) < 2:
            raise ValueError(f'{node.name}: matmul operands need rank >= 2, got {len(ls)} and {len(rs)}.')
        if int(ls[-1]) != int(rs[-2]):
            raise ValueError(f'{node.name}: matmul reduction extents differ: {ls[-1]} vs {rs[-2]}.')
        # the reference accepts only a rank-2 / broadcast RHS (matmul/resolver.py:440-463); here a batched
        # RHS is allowed when its leading axes equal the LHS's (independent products per leading index)
        if len(rs) > 2 and [int(x) for x in rs[:-2]] != [int(x) for x in ls[:-2]]:
            raise ValueError(f'{node.name}: batched matmul RHS leading axes {rs[:-2]} must equal the LHS leading axes '
                             f'{ls[:-2]}.')


@register_variant
class DenseGpuVariant(OpImplVariant):
    """Dense = int8 MFMA GEMM + int32 bias + shift/round/saturate + ReLU in one kernel."""

    variant_id = 'dense.b.r.gfx950.v1'
    op_type = 'dense'
    plevel = 10

    def matches(self, node, device) -> bool:
        return _bitwidths_supported(node, device)

    def resolve(self, node, _device, _directives=None) -> DenseConfig:
        precision = _resolve_numeric(node)
        precision['bias'] = _resolve_bias_dtype(node, precision)
        lhs, rhs = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        shift = resolve_accumulator_output_shift(lhs.precision, node.outputs[0].precision, rhs.precision)
        shift += _resolve_output_scale_shift(node)
        fused = node.traits.get('fused_activation')
        use_relu = ((fused.data.get('activation') if fused else '') or '').lower() == 'relu'
        lhs_perm = view_perm(node, lhs, 'inputs')
        w = np.asarray(rhs.data)
        per_channel = (node.directives or {}).get('shift_per_channel')
        if per_channel is not None:
            per_channel = tuple(int(v) for v in np.asarray(per_channel).reshape(-1))
        return DenseConfig(
            precision=precision,
            shift=int(shift),
            shift_per_channel=per_channel,
            accumulator_tag='acc64' if precision['acc'].format == 'int64' else 'acc32',
            rounding_mode=aie_rounding_token(precision['output']),
            flags=DenseFlags(use_relu=use_relu,
                             transpose_lhs=bool(lhs_perm is not None and lhs_perm[-1] != len(lhs_perm) - 1),
                             use_bias=bool(node.metadata.get('use_bias'))),
            n_in=int(w.shape[-2]),
            n_out=int(w.shape[-1]),
        )

    def validate_config(self, node, config: DenseConfig, _device) -> None:
        if config.shift < 0:
            raise ValueError(f'{node.name}: dense accumulator output shift must be non-negative, got {config.shift}.')
        top = 62 if config.accumulator_tag == 'acc64' else 31
        if config.shift > top:
            raise ValueError(f'{node.name}: dense accumulator output shift {config.shift} exceeds the '
                             f'{top + 1 if top == 31 else 64}-bit accumulator.')
        if config.shift_per_channel is not None:
            if len(config.shift_per_channel) != config.n_out:
                raise ValueError(f'{node.name}: shift_per_channel needs {config.n_out} entries, got '
                                 f'{len(config.shift_per_channel)}.')
            if min(config.shift_per_channel) < 0 or max(config.shift_per_channel) > top:
                raise ValueError(f'{node.name}: per-channel shifts must be in [0, {top}].')
        _check_out_format(node, config.precision['output'].format)
        lhs_perm = view_perm(node, input_tensor_for_role(node, 'lhs'), 'inputs')
        if not (is_identity(lhs_perm) or is_last_two_swap(lhs_perm)):
            raise ValueError(f'{node.name}: dense input does not support io_view permutation {lhs_perm}.')

    def quantize_weight_bias(self, inst):
        """Integer weights [K, N] and int32 bias at accumulator scale 2^(in_frac + w_frac)."""
        node = inst.node
        x, w = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        b = next((t for t in node.inputs if input_role(node, t.name) == 'bias'), None)
        wi = to_quant_intent(w.precision)
        W = quantize_to_int(w.data, wi.frac, wi.width, signed=wi.signed, rounding_mode=wi.rounding,
                            saturation_mode=w.precision.saturation)
        W = np.asarray(W).reshape((-1,) + tuple(np.asarray(w.data).shape[-2:]))[-1]
        bias = None
        if b is not None:
            bi = to_quant_intent(b.precision) if b.precision is not None else None
            acc_frac = to_quant_intent(x.precision).frac + wi.frac
            bias = quantize_to_int(np.asarray(b.data).reshape(-1), acc_frac, 32,
                                   signed=bi.signed if bi else True,
                                   rounding_mode=bi.rounding if bi else inst.config.precision['bias'].rounding,
                                   saturation_mode=b.precision.saturation if bi else inst.config.precision['bias'].saturation)
        if wi.width > 8:
            return W.astype(np.int16 if wi.signed else np.uint16), bias
        return W.astype(np.int8 if wi.signed else np.uint8), bias

    def pack(self, inst) -> Dict[str, Any]:
        import torch

        from .. import ops

        W, bias = self.quantize_weight_bias(inst)
        if W.dtype not in (np.int8, np.int16):
            raise ValueError(f'{inst.name}: dense weights must use a signed integer precision.')
        cfg = inst.config
        shifts = cfg.shift_per_channel if cfg.shift_per_channel is not None else cfg.shift
        dev = torch.device('cuda')
        packed = ops.pack_dense(torch.from_numpy(np.ascontiguousarray(W)).to(dev),
                                torch.from_numpy(bias.astype(np.int32)).to(dev) if bias is not None else None,
                                np.asarray(shifts, dtype=np.int32))
        return {'packed_weights': packed, 'weights_int': W, 'bias_int': bias}

    def get_artifacts(self, inst):
        return [{'name': 'weights', 'array': inst.artifacts.get('weights_int')},
                {'name': 'bias', 'array': inst.artifacts.get('bias_int')}]

    def run(self, inst, inputs):
        from .. import ops

        cfg = inst.config
        x = inputs[input_tensor_for_role(inst.node, 'lhs').name]
        # a transposed left operand (io_view perm) is read as stored: the kernel transposes its tiles (dense_bias_relu.cpp:95-101)
        y = ops.dense(x, inst.artifacts['packed_weights'], cfg.rounding_mode, relu=cfg.flags.use_relu,
                      out_kind=cfg.precision['output'].format, trans_a=cfg.flags.transpose_lhs)
        return {inst.node.outputs[0].name: y}


@register_variant
class MatmulGpuVariant(OpImplVariant):
    """Dynamic MatMul: batched int8 MFMA GEMM + shift/round/saturate; no bias, no ReLU."""

    variant_id = 'matmul.gfx950.v1'
    op_type = 'matmul'
    plevel = 10

    def matches(self, node, device) -> bool:
        return _bitwidths_supported(node, device)

    def resolve(self, node, _device, _directives=None) -> MatmulConfig:
        precision = _resolve_numeric(node)
        lhs, rhs = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        shift = resolve_accumulator_output_shift(lhs.precision, node.outputs[0].precision, rhs.precision)
        shift += _resolve_output_scale_shift(node)
        lp, rp = view_perm(node, lhs, 'inputs'), view_perm(node, rhs, 'inputs')
        return MatmulConfig(
            precision=precision,
            shift=int(shift),
            accumulator_tag='acc64' if precision['acc'].format == 'int64' else 'acc32',
            rounding_mode=aie_rounding_token(precision['output']),
            flags=MatmulFlags(transpose_lhs=bool(lp is not None and lp[-1] != len(lp) - 1),
                              transpose_rhs=bool(rp is not None and rp[-1] != len(rp) - 1)),
        )

    def validate_config(self, node, config: MatmulConfig, _device) -> None:
        rhs = input_tensor_for_role(node, 'rhs')
        rp = view_perm(node, rhs, 'inputs')
        if not (is_identity(rp) or is_last_two_swap(rp)):
            raise ValueError(f'{node.name}: matmul RHS does not support io_view permutation {rp}.')
        lp = view_perm(node, input_tensor_for_role(node, 'lhs'), 'inputs')
        if not (is_identity(lp) or is_last_two_swap(lp)):
            raise ValueError(f'{node.name}: matmul LHS does not support io_view permutation {lp}.')
        if not bool(config.precision['rhs'].signed):
            raise ValueError(f'{node.name}: matmul RHS must use a signed integer precision.')
        top = 62 if config.accumulator_tag == 'acc64' else 31
        if not 0 <= config.shift <= top:
            raise ValueError(f'{node.name}: matmul accumulator output shift must be in [0, {top}], got {config.shift}.')
        _check_out_format(node, config.precision['output'].format)

    def pack(self, inst) -> Dict[str, Any]:
        """A constant (non rank-2 or batched) RHS is quantised and uploaded once."""
        import torch

        rhs = input_tensor_for_role(inst.node, 'rhs')
        if not rhs.is_parameter:
            return {}
        q = to_quant_intent(rhs.precision)
        data = quantize_to_int(rhs.data, q.frac, q.width, signed=q.signed, rounding_mode=q.rounding,
                               saturation_mode=rhs.precision.saturation)
        return {'rhs_const': torch.from_numpy(np.ascontiguousarray(data.astype(np.int16 if q.width > 8 else np.int8))).cuda()}

    def run(self, inst, inputs):
        from .. import ops

        cfg, node = inst.config, inst.node
        lhs_t, rhs_t = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        a = inputs[lhs_t.name]
        b = inst.artifacts['rhs_const'] if rhs_t.is_parameter else inputs[rhs_t.name]
        ta = bool(cfg.flags.transpose_lhs)
        if ta and b.dim() == 2 and a.dim() > 2:  # shared rank-2 RHS: one product per leading index, each read as stored
            import torch

            lead = tuple(a.shape[:-2])
            a3 = a.reshape((-1,) + tuple(a.shape[-2:]))
            ys = [ops.matmul(a3[i], b, cfg.shift, cfg.rounding_mode, trans_b=cfg.flags.transpose_rhs,
                             out_kind=cfg.precision['output'].format, trans_a=True) for i in range(int(a3.shape[0]))]
            y = torch.stack(ys) if len(ys) != 1 else ys[0][None]
            return {node.outputs[0].name: y.reshape(lead + tuple(y.shape[-2:]))}
        rows_shape = tuple(a.shape[:-2]) + ((int(a.shape[-1]),) if ta else (int(a.shape[-2]),))
        out_shape = rows_shape + (int(b.shape[-2] if cfg.flags.transpose_rhs else b.shape[-1]),)
        if b.dim() == 2 and a.dim() > 2:
            a = a.reshape(-1, a.shape[-1])  # rank-2 RHS is shared by every leading index of the LHS
        # a transposed left operand (io_view perm) is read as stored: the kernel transposes its tiles (matmul.cpp:60-66)
        y = ops.matmul(a, b, cfg.shift, cfg.rounding_mode, trans_b=cfg.flags.transpose_rhs,
                       out_kind=cfg.precision['output'].format, trans_a=ta)
        return {node.outputs[0].name: y.reshape(out_shape)}
