"""Operator plugin API of the GPU backend.

Same lifecycle and registries as the reference (src/aie4ml/op_impls/base.py:19-88, registry.py:12-47,
family_registry.py:9-56): a FamilyResolver validates a node's structure and picks the first registered
variant whose matches(node, device) is true, by descending `plevel`; the variant's resolve() turns
tensor precisions, traits and directives into a frozen config of kernel constants, validate_config()
enforces the kernel ABI, pack() builds device-resident parameters. The AIE-only hooks (ports, staging,
footprint, template parameters) have no GPU meaning and are absent; run() is the GPU addition: it
launches the kernels for one resolved node.
"""

from __future__ import annotations

from typing import Any, ClassVar, Dict, List, Optional, Tuple


class OpImplVariant:
    variant_id: ClassVar[str] = ''
    op_type: ClassVar[str] = ''
    param_template: ClassVar[str] = ''  # no Jinja template: nothing is generated
    plevel: ClassVar[int] = 10          # higher value = higher selection priority

    def matches(self, _node, _device) -> bool:
        raise NotImplementedError

    def resolve(self, _node, _device, _directives: Optional[Dict[str, Any]] = None) -> Any:
        raise NotImplementedError

    def validate_config(self, _node, _config, _device) -> None:
        """Post-resolve verifier. Override to enforce kernel ABI rules."""

    def pack(self, _inst) -> Dict[str, Any]:
        return {}

    def get_artifacts(self, _inst) -> List[Dict[str, Any]]:
        return []

    def input_precision(self, config, role: str):
        return config.precision[role]

    def output_precision(self, config):
        return config.precision['output']

    def run(self, _inst, _inputs: Dict[str, Any]) -> Dict[str, Any]:
        """Execute the node on the GPU. `_inputs` maps input tensor name -> device tensor as stored by its
        producer; returns output tensor name -> device tensor."""
        raise NotImplementedError


class OpImplRegistry:
    def __init__(self):
        self._variants: Dict[str, List[OpImplVariant]] = {}

    def register(self, variant: OpImplVariant) -> None:
        self._variants.setdefault(variant.op_type, []).append(variant)

    def candidates(self, op_type: str) -> List[OpImplVariant]:
        return sorted(self._variants.get(op_type, []), key=lambda v: v.plevel, reverse=True)


_OP_IMPLS = OpImplRegistry()


def get_op_impl_registry() -> OpImplRegistry:
    return _OP_IMPLS


def register_variant(cls):
    _OP_IMPLS.register(cls())
    return cls


class FamilyResolver:
    """Structural validator + variant dispatcher for one op type."""

    op_type: ClassVar[str] = ''

    def validate_structure(self, _node, _device) -> None:
        raise NotImplementedError

    def resolve(self, node, device, directives=None) -> Tuple[Any, OpImplVariant]:
        self.validate_structure(node, device)
        for variant in get_op_impl_registry().candidates(self.op_type):
            if variant.matches(node, device):
                return variant.resolve(node, device, directives), variant
        raise ValueError(f'{node.name}: no {self.op_type} variant matches (generation={device.generation!r}).')


class FamilyResolverRegistry:
    def __init__(self):
        self._resolvers: Dict[str, FamilyResolver] = {}

    def register(self, op_type: str, resolver: FamilyResolver) -> None:
        self._resolvers[op_type] = resolver

    def get(self, op_type: str) -> FamilyResolver:
        try:
            return self._resolvers[op_type]
        except KeyError:
            raise NotImplementedError(f'No family resolver registered for op_type={op_type!r}.') from None


_FAMILIES = FamilyResolverRegistry()


def get_family_resolver_registry() -> FamilyResolverRegistry:
    return _FAMILIES


def family_resolver(*op_types: str):
    def decorator(cls):
        inst = cls()
        for op_type in op_types:
            _FAMILIES.register(str(op_type), inst)
        return cls

    return decorator


GPU_GENERATIONS = ('CDNA4',)


def is_gpu(device) -> bool:
    return getattr(device, 'generation', None) in GPU_GENERATIONS
