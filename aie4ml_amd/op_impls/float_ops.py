"""GPU variants of the reference's float compute path: Dense, MatMul and Add on bfloat16, float32 or fp8 e4m3 tensors.

In the reference the same variant classes serve both paths and branch on FloatIntent
(_DenseVariantBase.resolve, src/aie4ml/op_impls/families/matmul/dense.py:94-133: shift 0, accumulator
'accfloat', rounding 'conv_even'; _resolve_numeric, resolver.py:110-129: lhs, rhs and output must all be float;
_resolve_output_scale_shift :160-167: a folded scale is not implemented for float; _quantize_weight_bias,
dense.py:143-146: weights through pack_as_float, bias as float32; AddOpImplVariant, elementwise/add.py:83).
LayerNorm and Softmax have no float variant there (layer_norm.py:84-85, softmax.py:75-76) and none here.
"""

from __future__ import annotations

import torch

from dataclasses import dataclass
from typing import Any, Dict

import numpy as np

from ..aie_types import AIEDataType, is_float_intent
from ..ir import input_role, input_tensor_for_role
from .base import OpImplVariant, is_gpu, register_variant
from .dense import DenseFlags, MatmulFlags
from .precision import float_format_name, is_identity, is_last_two_swap, view_perm

GPU_FLOAT_FORMATS = ('bfloat16', 'float32', 'fp8_e4m3')


@dataclass(frozen=True)
class FloatDenseConfig:
    precision: Dict[str, Any]
    shift: int
    accumulator_tag: str
    rounding_mode: str
    flags: DenseFlags
    n_in: int
    n_out: int

    def __hash__(self):
        return id(self)


@dataclass(frozen=True)
class FloatMatmulConfig:
    precision: Dict[str, Any]
    shift: int
    accumulator_tag: str
    rounding_mode: str
    flags: MatmulFlags

    def __hash__(self):
        return id(self)


@dataclass(frozen=True)
class FloatAddConfig:
    precision: Dict[str, Any]
    shift: int
    accumulator_tag: str
    rounding_mode: str

    def __hash__(self):
        return id(self)


def float32_to_fp8_codes(array) -> np.ndarray:
    """float32 -> fp8 e4m3 codes (uint8), the integer recipe of the reference's _float32_to_fp8_scalar
    (matmul/common.py:262-276): round half away from zero at mantissa bit 20, bias 7, gradual underflow,
    magnitudes from 480 up give the code 0x7f."""
    bits = np.ascontiguousarray(np.asarray(array, dtype=np.float32)).view(np.uint32).astype(np.int64)
    h = (bits + 0x00080000) & 0xFFFFFFFF
    e, m, sign = (h & 0x7F800000) >> 23, h & 0x007FFFFF, (h & 0x80000000) >> 24
    normal = sign | (((e - 120) << 3) & 0x78) | (m >> 20)
    sub = sign | ((((0x00780000 + m) >> np.clip(140 - e, 0, 62)) + 1) >> 1)
    out = np.where(e > 135, sign | 0x7F, np.where(e > 120, normal, np.where(e > 116, sub, sign)))
    return (out & 0xFF).astype(np.uint8)


def fp8_codes_to_float32(codes) -> np.ndarray:
    """fp8 e4m3 codes -> float32 (bias 7, subnormals m * 2^-9, 0x7f / 0xff are NaN), exact."""
    c = np.asarray(codes, dtype=np.uint8).astype(np.int64)
    e, m = (c >> 3) & 0xF, c & 7
    mag = np.where(e == 0, m * 2.0 ** -9, (1.0 + m / 8.0) * np.exp2(e - 7.0))
    mag = np.where((e == 15) & (m == 7), np.nan, mag)
    return np.where(c & 0x80, -mag, mag).astype(np.float32)


def pack_as_float(array, fmt: str) -> np.ndarray:
    """Parameter data -> values of the storage format, as float32 (pack_as_float, matmul/common.py:253-284:
    bfloat16 keeps the upper 16 bits of the float32 pattern, i.e. truncates; fp8 goes through the packer's
    integer recipe)."""
    f32 = np.ascontiguousarray(np.asarray(array, dtype=np.float32))
    if fmt == 'bfloat16':
        return ((f32.view(np.uint32) >> 16) << 16).view(np.float32)
    if fmt == 'float32':
        return f32
    if fmt == 'fp8_e4m3':
        return fp8_codes_to_float32(float32_to_fp8_codes(f32))
    raise NotImplementedError(f'float format {fmt!r} has no GPU kernel (bfloat16, float32 and fp8_e4m3 do).')


def _torch_dtype(fmt: str):
    import torch

    return {'bfloat16': torch.bfloat16, 'float32': torch.float32, 'fp8_e4m3': torch.float8_e4m3fn}[fmt]


def to_device_float(array, fmt: str):
    """float32 host values that are exact in `fmt` -> device tensor of that format."""
    import torch

    if fmt == 'fp8_e4m3':  # by code, so that the packer's recipe (not the library's cast) decides every bit
        return torch.from_numpy(float32_to_fp8_codes(array)).cuda().view(torch.float8_e4m3fn)
    return torch.from_numpy(np.ascontiguousarray(array, dtype=np.float32)).cuda().to(_torch_dtype(fmt))


def _float_precision(node, tensors) -> Dict[str, AIEDataType]:
    if any(t.precision is None for t in tensors.values()):
        raise ValueError(f'{node.name}: missing precision metadata for {node.op_type}.')
    if not all(is_float_intent(t.precision) for t in tensors.values()):
        raise ValueError(f'{node.name}: float {node.op_type} requires lhs/rhs/output to share float precision.')
    fmts = {k: float_format_name(t.precision) for k, t in tensors.items()}
    if len(set(fmts.values())) != 1:
        raise ValueError(f'{node.name}: float {node.op_type} requires lhs/rhs/output to share float precision.')
    fmt = fmts['lhs']
    if fmt not in GPU_FLOAT_FORMATS:
        raise NotImplementedError(f'{node.name}: float format {fmt!r} has no GPU kernel.')
    precision = {k: AIEDataType(format=fmt) for k in tensors}
    precision['acc'] = AIEDataType(format='accfloat')
    return precision


def _is_float_node(node, device) -> bool:
    if not is_gpu(device):
        return False
    lhs = input_tensor_for_role(node, 'lhs')
    return lhs.precision is not None and is_float_intent(lhs.precision)


def _reject_output_scale(node) -> None:
    if node.traits.get('output_scale') is not None:
        raise NotImplementedError(f'{node.name}: fused output scaling is not implemented for float MatMul-family ops.')


@register_variant
class DenseFloatGpuVariant(OpImplVariant):
    """Float Dense = bf16 / fp32 MFMA GEMM from a float32 accumulator that starts at the bias, ReLU, one rounding."""

    variant_id = 'dense.b.r.float.gfx950.v1'
    op_type = 'dense'
    plevel = 10

    def matches(self, node, device) -> bool:
        return _is_float_node(node, device)

    def resolve(self, node, _device, _directives=None) -> FloatDenseConfig:
        lhs, rhs = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        precision = _float_precision(node, {'lhs': lhs, 'rhs': rhs, 'output': node.outputs[0]})
        precision['bias'] = AIEDataType(format='float32')
        _reject_output_scale(node)
        fused = node.traits.get('fused_activation')
        use_relu = ((fused.data.get('activation') if fused else '') or '').lower() == 'relu'
        lhs_perm = view_perm(node, lhs, 'inputs')
        w = np.asarray(rhs.data)
        return FloatDenseConfig(precision=precision, shift=0, accumulator_tag='accfloat', rounding_mode='conv_even',
                                flags=DenseFlags(use_relu=use_relu,
                                                 transpose_lhs=bool(lhs_perm is not None and lhs_perm[-1] != len(lhs_perm) - 1),
                                                 use_bias=bool(node.metadata.get('use_bias'))),
                                n_in=int(w.shape[-2]), n_out=int(w.shape[-1]))

    def validate_config(self, node, config, _device) -> None:
        lhs_perm = view_perm(node, input_tensor_for_role(node, 'lhs'), 'inputs')
        if not (is_identity(lhs_perm) or is_last_two_swap(lhs_perm)):
            raise ValueError(f'{node.name}: dense input does not support io_view permutation {lhs_perm}.')

    def pack(self, inst) -> Dict[str, Any]:
        import torch

        from .. import ops

        node, fmt = inst.node, inst.config.precision['rhs'].format
        w = input_tensor_for_role(node, 'rhs')
        b = next((t for t in node.inputs if input_role(node, t.name) == 'bias'), None)
        W = pack_as_float(w.data, fmt)
        W = W.reshape((-1,) + tuple(W.shape[-2:]))[-1]
        bias = np.asarray(b.data, dtype=np.float32).reshape(-1) if b is not None else None
        packed = ops.pack_dense_float(to_device_float(W, fmt), torch.from_numpy(bias).cuda() if bias is not None else None)
        return {'packed_weights': packed, 'weights_float': W, 'bias_float': bias}

    def get_artifacts(self, inst):
        return [{'name': 'weights', 'array': inst.artifacts.get('weights_float')},
                {'name': 'bias', 'array': inst.artifacts.get('bias_float')}]

    def run(self, inst, inputs):
        from .. import ops

        cfg = inst.config
        x = inputs[input_tensor_for_role(inst.node, 'lhs').name]
        # a transposed input (io_view perm) is read as stored: the kernel transposes its tiles (dense_bias_relu.cpp:95-101)
        return {inst.node.outputs[0].name: ops.dense_float(x, inst.artifacts['packed_weights'], relu=cfg.flags.use_relu,
                                                           trans_a=bool(cfg.flags.transpose_lhs))}


@register_variant
class MatmulFloatGpuVariant(OpImplVariant):
    """Float dynamic MatMul: batched bf16 / fp32 MFMA GEMM, one rounding to the operand format."""

    variant_id = 'matmul.float.gfx950.v1'
    op_type = 'matmul'
    plevel = 10

    def matches(self, node, device) -> bool:
        return _is_float_node(node, device)

    def resolve(self, node, _device, _directives=None) -> FloatMatmulConfig:
        lhs, rhs = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        precision = _float_precision(node, {'lhs': lhs, 'rhs': rhs, 'output': node.outputs[0]})
        _reject_output_scale(node)
        lp, rp = view_perm(node, lhs, 'inputs'), view_perm(node, rhs, 'inputs')
        return FloatMatmulConfig(precision=precision, shift=0, accumulator_tag='accfloat', rounding_mode='conv_even',
                                 flags=MatmulFlags(transpose_lhs=bool(lp is not None and lp[-1] != len(lp) - 1),
                                                   transpose_rhs=bool(rp is not None and rp[-1] != len(rp) - 1)))

    def validate_config(self, node, config, _device) -> None:
        for role in ('lhs', 'rhs'):
            perm = view_perm(node, input_tensor_for_role(node, role), 'inputs')
            if not (is_identity(perm) or is_last_two_swap(perm)):
                raise ValueError(f'{node.name}: matmul {role.upper()} does not support io_view permutation {perm}.')

    def pack(self, inst) -> Dict[str, Any]:
        rhs = input_tensor_for_role(inst.node, 'rhs')
        if not rhs.is_parameter:
            return {}
        fmt = inst.config.precision['rhs'].format
        return {'rhs_const': to_device_float(pack_as_float(rhs.data, fmt), fmt)}

    def run(self, inst, inputs):
        from .. import ops

        cfg, node = inst.config, inst.node
        lhs_t, rhs_t = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        a = inputs[lhs_t.name]
        b = inst.artifacts['rhs_const'] if rhs_t.is_parameter else inputs[rhs_t.name]
        ta = bool(cfg.flags.transpose_lhs)
        n_out = int(b.shape[-2] if cfg.flags.transpose_rhs else b.shape[-1])
        # a transposed left operand (io_view perm) is read as stored: the kernel transposes its tiles (matmul.cpp:60-66)
        if ta and b.dim() == 2 and a.dim() > 2:  # shared rank-2 RHS: one product per leading index
            lead = tuple(a.shape[:-2])
            a3 = a.reshape((-1,) + tuple(a.shape[-2:]))
            y = torch.empty((a3.shape[0], int(a.shape[-1]), n_out), dtype=a.dtype, device=a.device)
            for i in range(int(a3.shape[0])):
                ops.matmul_float(a3[i], b, trans_b=cfg.flags.transpose_rhs, trans_a=True, out=y[i])
            return {node.outputs[0].name: y.reshape(lead + tuple(y.shape[-2:]))}
        out_shape = tuple(a.shape[:-2]) + (int(a.shape[-1] if ta else a.shape[-2]), n_out)
        if b.dim() == 2 and a.dim() > 2:
            a = a.reshape(-1, a.shape[-1])
        y = ops.matmul_float(a, b, trans_b=cfg.flags.transpose_rhs, trans_a=ta)
        return {node.outputs[0].name: y.reshape(out_shape)}


@register_variant
class AddFloatGpuVariant(OpImplVariant):
    variant_id = 'add.float.gfx950.v1'
    op_type = 'add'
    plevel = 10

    def matches(self, node, device) -> bool:
        return _is_float_node(node, device)

    def resolve(self, node, _device, _directives=None) -> FloatAddConfig:
        lhs, rhs = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        precision = _float_precision(node, {'lhs': lhs, 'rhs': rhs, 'output': node.outputs[0]})
        return FloatAddConfig(precision=precision, shift=0, accumulator_tag='accfloat', rounding_mode='conv_even')

    def run(self, inst, inputs):
        from .. import ops

        node = inst.node
        a = inputs[input_tensor_for_role(node, 'lhs').name]
        b = inputs[input_tensor_for_role(node, 'rhs').name]
        return {node.outputs[0].name: ops.add_float(a, b)}
