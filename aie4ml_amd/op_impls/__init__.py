"""Operator variants of the GPU backend. Importing the package registers every family and variant."""

from . import dense, elementwise, float_ops, layernorm, softmax  # noqa: F401  (registration side effects)
from .base import (FamilyResolver, OpImplVariant, family_resolver, get_family_resolver_registry,
                   get_op_impl_registry, register_variant)

__all__ = ['FamilyResolver', 'OpImplVariant', 'family_resolver', 'get_family_resolver_registry',
           'get_op_impl_registry', 'register_variant']
