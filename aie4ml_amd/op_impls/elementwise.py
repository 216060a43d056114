"""GPU variant of elementwise Add (AddOpImplVariant.resolve, src/aie4ml/op_impls/families/elementwise/
add.py:57-164; structural rules from elementwise/resolver.py:14-33)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict

from ..aie_types import is_float_intent
from ..ir import input_tensor_for_role
from .base import FamilyResolver, OpImplVariant, family_resolver, is_gpu, register_variant
from .precision import aie_rounding_token, resolve_accumulator_output_shift, resolve_exact_storage_dtype, view_shape


@dataclass(frozen=True)
class AddConfig:
    precision: Dict[str, Any]
    shift: int
    accumulator_tag: str
    rounding_mode: str

    def __hash__(self):
        return id(self)


@family_resolver('add')
class AddFamilyResolver(FamilyResolver):
    op_type = 'add'

    def validate_structure(self, node, _device) -> None:
        lhs, rhs = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        ls = tuple(int(x) for x in view_shape(node, lhs, 'inputs'))
        rs = tuple(int(x) for x in view_shape(node, rhs, 'inputs'))
        if len(ls) < 2:
            raise ValueError(f'{node.name}: elementwise Add requires rank>=2, got {len(ls)}.')
        if ls != rs:
            raise ValueError(f'{node.name}: elementwise Add requires exact-shape inputs, got {ls} and {rs}.')
        tensors = (lhs, rhs, node.outputs[0])
        if any(t.precision is None for t in tensors):
            raise ValueError(f'{node.name}: missing precision metadata for add.')
        if any(is_float_intent(t.precision) for t in tensors):
            # float Add: all three tensors float (elementwise/resolver.py:26-28); the float variant checks formats
            if not all(is_float_intent(t.precision) for t in tensors):
                raise ValueError(f'{node.name}: elementwise Add requires lhs/rhs/output to use the same storage type.')
            return
        kinds = [resolve_exact_storage_dtype(t.precision, namespace=ns, layer_name=node.name)
                 for t, ns in zip(tensors, ('lhs', 'rhs', 'output'))]
        if kinds[0] != kinds[1] or kinds[0] != kinds[2]:
            raise ValueError(f'{node.name}: elementwise Add requires lhs/rhs/output to use the same storage type.')


@register_variant
class AddGpuVariant(OpImplVariant):
    variant_id = 'add.gfx950.v1'
    op_type = 'add'
    plevel = 10

    def matches(self, node, device) -> bool:
        lhs = input_tensor_for_role(node, 'lhs')
        return is_gpu(device) and not is_float_intent(lhs.precision)

    def resolve(self, node, _device, _directives=None) -> AddConfig:
        lhs, rhs = input_tensor_for_role(node, 'lhs'), input_tensor_for_role(node, 'rhs')
        precision = {
            'lhs': resolve_exact_storage_dtype(lhs.precision, namespace='lhs', layer_name=node.name),
            'rhs': resolve_exact_storage_dtype(rhs.precision, namespace='rhs', layer_name=node.name),
            'output': resolve_exact_storage_dtype(node.outputs[0].precision, namespace='output', layer_name=node.name),
        }
        return AddConfig(precision=precision,
                         shift=resolve_accumulator_output_shift(lhs.precision, node.outputs[0].precision),
                         accumulator_tag='acc32',
                         rounding_mode=aie_rounding_token(precision['output']))

    def validate_config(self, node, config: AddConfig, _device) -> None:
        if config.precision['lhs'].format not in ('int8', 'uint8', 'int16'):
            raise NotImplementedError(f'{node.name}: GPU Add runs on int8, uint8 or int16 tensors, not '
                                      f'{config.precision["lhs"].format!r}.')

    def run(self, inst, inputs):
        from .. import ops

        node, cfg = inst.node, inst.config
        a = inputs[input_tensor_for_role(node, 'lhs').name]
        b = inputs[input_tensor_for_role(node, 'rhs').name]
        return {node.outputs[0].name: ops.add(a, b, cfg.shift, cfg.rounding_mode)}
